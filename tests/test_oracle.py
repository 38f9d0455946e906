"""Pins the CPU oracle (NumPy and C restatements) without running the reference.

Every check is chosen so that a plausible mistake fails it: wrong field order or
arithmetic shift (known-answer words), a second rounding or a fused zero-point
(exhaustive float64 closed form), a transposed operand (non-square one-hot
readback), a reassociated sum (order-sensitive hand-computed case).
"""
import numpy as np
import pytest

from oracle import c_oracle, wq_oracle as O


# ------------------------------------------------------------------ float16 conversions (C)
def test_c_f16_to_f32_all_values():
    got = c_oracle.f16_to_f32_all()
    want = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    nan = np.isnan(want)  # a signalling NaN is quieted when returned by value: compare NaNs as a class
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


def test_c_f32_to_f16_rne():
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    # every float16 value, every midpoint between neighbours and one ulp32 either side
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    edge = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                           np.array([65504, 65519.996, 65520, 65536, 1e30, np.inf, 2.0**-24, 2.0**-25,
                                     np.nextafter(np.float32(2.0**-25), np.float32(1)), 2.0**-26, 0.0],
                                    dtype=np.float32)])
    vals = np.concatenate([bits.view(np.float32), edge, -edge])
    got = c_oracle.f32_to_f16(vals)
    with np.errstate(all="ignore"):
        want = vals.astype(np.float16)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])


# ------------------------------------------------------------------ unpack
def _bitwalk_fields(word: int, bits: int):
    """Independent statement: peel fields off the least-significant end with Python ints."""
    out = []
    for _ in range(32 // bits):
        out.append(word % (1 << bits))
        word //= 1 << bits
    return out


@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_unpack_known_answers(impl):
    wq4 = np.array([[0x76543210, 0xFEDCBA98], [0x0000000F, 0xF0000000]], dtype=np.uint32)
    want4 = np.array([[0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15],
                      [15, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 15]], dtype=np.uint8)
    wq8 = np.array([[0x80FF7F01, 0x000000FE]], dtype=np.uint32)
    want8 = np.array([[1, 127, -1, -128, -2, 0, 0, 0]], dtype=np.int8)
    if impl == "numpy":
        got4, got8 = O.unpack_q4(wq4), O.unpack_q8(wq8)
    else:
        got4, got8 = c_oracle.unpack(wq4, 4), c_oracle.unpack(wq8, 8)
    assert got4.dtype == np.uint8 and np.array_equal(got4, want4)
    assert got8.dtype == np.int8 and np.array_equal(got8, want8)


@pytest.mark.parametrize("bits", [4, 8])
def test_unpack_every_field_value_and_position(bits):
    per = 32 // bits
    words = [v << (bits * pos) for pos in range(per) for v in range(1 << bits)]
    rng = np.random.default_rng(2)
    words += [int(v) for v in rng.integers(0, 2**32, size=4096, dtype=np.uint64)]
    wq = np.array(words, dtype=np.uint32).reshape(-1, 1)
    want = np.array([_bitwalk_fields(w, bits) for w in words], dtype=np.int64)
    if bits == 8:
        want = np.where(want >= 128, want - 256, want)  # two's-complement truncation to int8
    for got in (O.unpack_q4(wq) if bits == 4 else O.unpack_q8(wq), c_oracle.unpack(wq, bits)):
        assert np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("bits", [4, 8])
def test_pack_unpack_roundtrip(bits):
    rng = np.random.default_rng(3)
    wq = rng.integers(0, 2**32, size=(5, 24), dtype=np.uint64).astype(np.uint32)
    if bits == 4:
        assert np.array_equal(O.pack_q4(O.unpack_q4(wq)), wq)
    else:
        assert np.array_equal(O.pack_q8(O.unpack_q8(wq)), wq)


# ------------------------------------------------------------------ dequantize (bit exact, exhaustive)
def _bits_equal_nan_aware(a, b):
    na, nb = np.isnan(a), np.isnan(b)
    return np.array_equal(na, nb) and np.array_equal(a.view(np.uint16)[~na], b.view(np.uint16)[~nb])


@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_dequant_q4_exhaustive_closed_form(impl):
    """All 16 field values x all 65536 scale bit patterns; closed form = one rounding of the exact product."""
    scales = np.arange(65536, dtype=np.uint16).view(np.float16)
    # row r holds field value r in every position: K = 65536*32 would be large, so use group 32 with
    # one distinct scale per group and all 32 entries of the group equal to r.
    n_groups = 65536
    for r in range(16):
        word = sum(r << (4 * i) for i in range(8))
        wq = np.full((1, n_groups * 4), word, dtype=np.uint32)
        s = scales.reshape(1, n_groups)
        got = O.dequant_q4f16(wq, s) if impl == "numpy" else c_oracle.dequant(wq, s, 4, 32)
        with np.errstate(all="ignore"):
            want = (np.float64(r - 7) * scales.astype(np.float64)).astype(np.float16)
        assert _bits_equal_nan_aware(got.reshape(n_groups, 32)[:, 0], want), r
        assert _bits_equal_nan_aware(got.reshape(n_groups, 32)[:, 31], want), r


@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_dequant_q8_exhaustive_closed_form(impl):
    scales = np.arange(65536, dtype=np.uint16).view(np.float16)
    for r in list(range(-128, 128, 5)) + [-127, -1, 0, 1, 127]:
        word = sum((r & 0xFF) << (8 * i) for i in range(4))
        wq = np.full((1, 65536 * 32), word, dtype=np.uint32)  # group 128 = 32 words
        s = scales.reshape(1, 65536)
        got = O.dequant_q8f16(wq, s) if impl == "numpy" else c_oracle.dequant(wq, s, 8, 128)
        with np.errstate(all="ignore"):
            want = (np.float64(r) * scales.astype(np.float64)).astype(np.float16)
        assert _bits_equal_nan_aware(got.reshape(65536, 128)[:, 77], want), r


def test_dequant_group_indexing_and_layout():
    """Distinct power-of-two scales per (row, group): a wrong group index or row stride shows up exactly."""
    n, k, g = 3, 96, 32
    w = (np.arange(n * k).reshape(n, k) * 7 + 3) % 16
    s = (2.0 ** np.arange(n * (k // g))).reshape(n, k // g).astype(np.float16)
    want = ((w - 7) * np.repeat(s.astype(np.float64), g, axis=1)).astype(np.float16)
    wq = O.pack_q4(w)
    assert np.array_equal(O.dequant_q4f16(wq, s), want)
    assert np.array_equal(c_oracle.dequant(wq, s, 4, g), want)


# ------------------------------------------------------------------ matmul
@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_matmul_order_sensitive_known_answer(impl):
    """products 2^24, 1, -2^24, 1: sequential float32 from 0 gives 1 (true sum 2, reversed order gives 2)."""
    x = np.array([[4096, 1, -4096, 1]], dtype=np.float16)
    wd = np.array([[4096, 1, 4096, 1], [1, 1, 1, 1]], dtype=np.float16)
    f = O.matmul_f32acc if impl == "numpy" else c_oracle.matmul_f32acc
    y = f(x, wd)
    assert y.dtype == np.float32 and y.shape == (1, 2)
    assert y[0, 0] == 1.0 and y[0, 1] == 2.0


@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_matmul_products_are_float32_not_float16(impl):
    """(1+2^-10)^2 needs 21 significand bits: a float16 product or accumulator would lose the 2^-20 term."""
    a = np.float16(1 + 2.0**-10)
    f = O.matmul_f32acc if impl == "numpy" else c_oracle.matmul_f32acc
    y = f(np.array([[a]], dtype=np.float16), np.array([[a]], dtype=np.float16))
    assert y[0, 0] == np.float32(1 + 2.0**-9 + 2.0**-20)


@pytest.mark.parametrize("impl", ["numpy", "c"])
@pytest.mark.parametrize("bits,group", [(4, 32), (8, 128)])
def test_path_integer_special_case_is_exact(impl, bits, group):
    """S == 1 and small integer x: every partial sum is an integer < 2^11, so y equals the int64 matmul."""
    rng = np.random.default_rng(4)
    m, n, k = 3, 5, 2 * group
    x = rng.integers(-1, 2, size=(m, k)).astype(np.float16)
    if bits == 4:
        w = rng.integers(0, 16, size=(n, k))
        wq, centred = O.pack_q4(w), w - 7
    else:
        w = rng.integers(-3, 4, size=(n, k))
        wq, centred = O.pack_q8(w), w
    s = np.ones((n, k // group), dtype=np.float16)
    want = x.astype(np.int64) @ centred.T.astype(np.int64)
    assert np.abs(want).max() < 2048
    f = O.wq_matmul if impl == "numpy" else c_oracle.wq_matmul
    got = f(x, wq, s, bits, group)
    assert got.dtype == np.float16 and np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_path_one_hot_reads_back_dequantized_column(impl):
    """x = e_j (M != N != K): y[j', :] must be Wd[:, j'] -- catches transposed operands and strides."""
    x_, wq, s, g = O.make_case(5, 1, 6, 64, 4)
    picks = [0, 9, 33, 63]
    x = np.zeros((len(picks), 64), dtype=np.float16)
    for r, j in enumerate(picks):
        x[r, j] = 1
    wd = O.dequant_q4f16(wq, s)
    f = O.wq_matmul if impl == "numpy" else c_oracle.wq_matmul
    got = f(x, wq, s, 4, g)
    assert got.shape == (4, 6)
    assert np.array_equal(got.view(np.uint16), wd[:, picks].T.view(np.uint16))


@pytest.mark.parametrize("bits,m,n,k", [(4, 1, 64, 256), (4, 5, 33, 352), (8, 2, 40, 384)])
def test_c_and_numpy_oracles_agree_bitwise_and_track_float64(bits, m, n, k):
    x, wq, s, g = O.make_case(6, m, n, k, bits)
    y_np = O.wq_matmul(x, wq, s, bits, g)
    y_c = c_oracle.wq_matmul(x, wq, s, bits, g)
    y_c4 = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=4)
    assert np.array_equal(y_np.view(np.uint16), y_c.view(np.uint16))
    assert np.array_equal(y_c.view(np.uint16), y_c4.view(np.uint16))
    wd = O.dequant(wq, s, bits, g).astype(np.float64)
    y64 = x.astype(np.float64) @ wd.T
    mag = np.abs(x.astype(np.float64)) @ np.abs(wd).T
    # sequential float32 sum: |err| <= K * 2^-24 * sum|terms|, plus half an ulp of the float16 result
    bound = k * 2.0**-24 * mag + 2.0**-11 * np.abs(y64) + 2.0**-24
    assert np.all(np.abs(y_np.astype(np.float64) - y64) <= bound)


def test_make_case_distributions():
    x, wq, s, g = O.make_case(0, 2, 64, 4096, 4)
    assert g == 32 and wq.shape == (64, 512) and s.shape == (64, 128) and x.dtype == np.float16
    w = O.unpack_q4(wq)
    assert w.min() == 0 and w.max() == 15 and abs(w.mean() - 7.5) < 0.05
    assert 0.00499 <= float(s.min()) and float(s.max()) <= 0.02001
    x, wq, s, g = O.make_case(0, 1, 64, 5120, 8)
    w = O.unpack_q8(wq)
    assert g == 128 and w.min() == -127 and w.max() == 127
    assert 0.00199 <= float(s.min()) and float(s.max()) <= 0.01001


# ------------------------------------------------------------------ fused tail: float16 add, relu
def _f16(bits):
    return np.array(bits, dtype=np.uint16).view(np.float16)


def _add_both(a, b):
    """a + b through both restatements (the C one via its epilogue with a as y and b as bias)."""
    a = np.asarray(a, dtype=np.float16).reshape(1, -1)
    b = np.asarray(b, dtype=np.float16).reshape(-1)
    got_np = O.add_f16(a, b.reshape(1, -1))
    got_c = c_oracle.epilogue(a, bias=b)
    return got_np.reshape(-1), got_c.reshape(-1)


def test_f16_add_known_answers():
    """Ties go to even, sums past 65504 + 16 overflow, signed zeros and infinities follow IEEE 754."""
    cases = [
        (2048.0, 1.0, 2048.0),            # tie: 2049 lies between 2048 (even) and 2050
        (2048.0, 3.0, 2052.0),            # tie: 2051 -> 2052 (even significand)
        (1.0, 2.0**-11, 1.0),             # half an ulp above 1: tie to even
        (1.0, 3 * 2.0**-11, 1.0 + 2.0**-9),
        (1.0, 2.0**-11 + 2.0**-21, 1.0 + 2.0**-10),   # the next float16 above 2^-11: just past the tie
        (65504.0, 8.0, 65504.0),
        (65504.0, 16.0, np.inf),          # tie at 65520 rounds to the even neighbour 2^16 = overflow
        (-65504.0, -16.0, -np.inf),
        (6.0e-8, 6.0e-8, 1.2e-7),         # subnormal + subnormal is exact (both are 2^-24)
        (1024.0, -1023.5, 0.5),           # exact cancellation
        (0.1, 0.2, 0.2998046875),         # f16(0.1) + f16(0.2) = 0.29998779296875 -> 0.2998046875
    ]
    a = np.array([c[0] for c in cases], dtype=np.float16)
    b = np.array([c[1] for c in cases], dtype=np.float16)
    want = np.array([c[2] for c in cases], dtype=np.float16)
    for got in _add_both(a, b):
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (got, want)
    # signed zeros: (+0) + (-0) = +0, (-0) + (-0) = -0, x + (-x) = +0; inf - inf is NaN
    a = _f16([0x0000, 0x8000, 0x3C00, 0x7C00])
    b = _f16([0x8000, 0x8000, 0xBC00, 0xFC00])
    for got in _add_both(a, b):
        assert list(got.view(np.uint16)[:3]) == [0x0000, 0x8000, 0x0000] and np.isnan(got[3])


def test_f16_add_against_exact_rationals():
    """Independent check of the rounding: exact sums as fractions, nearest-even by search in the
    sorted table of all finite float16 values (no floating-point arithmetic on the checking side)."""
    import bisect
    from fractions import Fraction

    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    finite = halves[np.isfinite(halves) & ~((halves == 0) & np.signbit(halves))]  # drop -0: one zero in the table
    order = np.argsort(finite.astype(np.float64), kind="stable")
    table = finite[order]
    fracs = [Fraction(float(h)) for h in table]
    big = Fraction(65520)  # halfway between 65504 and 2^16

    def nearest(fr):
        if fr >= big:
            return np.float16(np.inf)
        if fr <= -big:
            return np.float16(-np.inf)
        i = bisect.bisect_left(fracs, fr)
        cands = [j for j in (i - 1, i) if 0 <= j < len(fracs)]
        dist = [abs(fracs[j] - fr) for j in cands]
        if len(cands) == 2 and dist[0] == dist[1]:
            j = cands[0] if (int(table[cands[0]].view(np.uint16)) & 1) == 0 else cands[1]
        else:
            j = cands[int(np.argmin(dist))]
        return table[j]

    rng = np.random.default_rng(42)
    bits_a = rng.integers(0, 65536, size=3000).astype(np.uint16)
    bits_b = rng.integers(0, 65536, size=3000).astype(np.uint16)
    # add pairs with nearby exponents (where rounding ties actually occur) and opposite signs
    near = rng.integers(0x3000, 0x4800, size=3000).astype(np.uint16)
    bits_a = np.concatenate([bits_a, near, near])
    bits_b = np.concatenate([bits_b, near + rng.integers(0, 64, size=3000).astype(np.uint16),
                             (near ^ 0x8000) + rng.integers(0, 3, size=3000).astype(np.uint16)])
    a, b = bits_a.view(np.float16), bits_b.view(np.float16)
    ok = np.isfinite(a) & np.isfinite(b)
    a, b = a[ok], b[ok]
    got_np, got_c = _add_both(a, b)
    for i in range(a.size):
        exact = Fraction(float(a[i])) + Fraction(float(b[i]))
        want = nearest(exact)
        if exact == 0:
            assert got_np[i] == 0 and got_c[i] == 0
            continue
        assert got_np[i].view(np.uint16) == want.view(np.uint16), (a[i], b[i])
        assert got_c[i].view(np.uint16) == want.view(np.uint16), (a[i], b[i])


def test_relu_special_values_and_epilogue_order():
    t = _f16([0x8000, 0x0000, 0x0001, 0x8001, 0x7C00, 0xFC00, 0x7E00, 0xFE00, 0x3C00, 0xBC00])
    want = [0x0000, 0x0000, 0x0001, 0x0000, 0x7C00, 0x0000, 0x0000, 0x0000, 0x3C00, 0x0000]
    assert list(O.relu_f16(t).view(np.uint16)) == want
    assert list(c_oracle.epilogue(t.reshape(1, -1), activation="relu").view(np.uint16).reshape(-1)) == want
    # order: bias before relu, residual after: y = -1, bias = +0.5 -> relu(-0.5) = 0 -> + residual 2 = 2;
    # any other order gives 1.5 (relu last on -1+0.5+2) or 2.5 (relu first)
    y = np.array([[-1.0]], dtype=np.float16)
    for impl in (O, c_oracle):
        out = impl.epilogue(y, bias=np.array([0.5], dtype=np.float16), activation="relu",
                            residual=np.array([[2.0]], dtype=np.float16))
        assert float(out[0, 0]) == 2.0
    # bias broadcasts over rows, residual is element-wise
    y = np.zeros((2, 3), dtype=np.float16)
    b = np.array([1, 2, 3], dtype=np.float16)
    r = np.array([[10, 20, 30], [40, 50, 60]], dtype=np.float16)
    for impl in (O, c_oracle):
        assert np.array_equal(impl.epilogue(y, bias=b, residual=r), r + b[None, :])
    with pytest.raises(ValueError):
        O.epilogue(y, activation="tanh")


@pytest.mark.parametrize("bits,m,n,k", [(4, 3, 40, 128), (8, 5, 24, 256)])
def test_fused_path_is_epilogue_of_plain_path(bits, m, n, k):
    x, wq, s, g = O.make_case(8, m, n, k, bits)
    rng = np.random.default_rng(3)
    bias = rng.standard_normal(n).astype(np.float16)
    res = rng.standard_normal((m, n)).astype(np.float16)
    plain = O.wq_matmul(x, wq, s, bits, g)
    for act in (None, "relu"):
        a = O.wq_matmul_fused(x, wq, s, bits, g, bias, act, res)
        c = c_oracle.wq_matmul_fused(x, wq, s, bits, g, bias, act, res)
        assert np.array_equal(a.view(np.uint16), c.view(np.uint16))
        t = plain.astype(np.float64) + bias.astype(np.float64)[None, :]
        t = t.astype(np.float16)
        if act:
            t = np.maximum(t, np.float16(0))
        want = (t.astype(np.float64) + res.astype(np.float64)).astype(np.float16)
        assert np.array_equal(a.view(np.uint16), want.view(np.uint16))


# ---------------------------------------------------------------- tile-major weight layout
@pytest.mark.parametrize("bits,n,k", [(4, 16, 256), (4, 37, 512), (8, 16, 128), (8, 50, 384)])
def test_tile_major_layout_definition_and_round_trip(bits, n, k):
    """The loop restatement places known chunks where the definition says, pads whole tiles with
    zeros, and the independently written inverse (reshape / transpose) returns the input."""
    rng = np.random.default_rng(bits * 1000 + n)
    group = 32 if bits == 4 else 128
    wq = rng.integers(0, 2**32, size=(n, k * bits // 32), dtype=np.uint64).astype(np.uint32)
    s = rng.standard_normal((n, k // group)).astype(np.float16)
    wt, st = O.tile_weights(wq, s, bits)
    rows = (n + 15) // 16 * 16
    assert wt.shape == (rows, wq.shape[1]) and st.shape == (rows, s.shape[1])
    flat, nsuper = wt.reshape(-1), k * bits // 8 // 128
    # hand-computed positions (in 32-bit words): row 0 chunk 0 first; row 1 chunk 0 one lane (4 words) later;
    # row 0 chunk 1 (d = 1) one 1 KB block later; row 0 chunk 2 (kq = 1) sixteen lanes later
    assert np.array_equal(flat[0:4], wq[0, 0:4]) and np.array_equal(flat[4:8], wq[1, 0:4])
    assert np.array_equal(flat[256:260], wq[0, 4:8]) and np.array_equal(flat[64:68], wq[0, 8:12])
    if nsuper > 1:  # row 0, chunk 8 = super step 1: two 1 KB blocks further
        assert np.array_equal(flat[512:516], wq[0, 32:36])
    if n > 16:      # row 16 = tile 1: after all super steps of tile 0
        assert np.array_equal(flat[nsuper * 512:nsuper * 512 + 4], wq[16, 0:4])
    sf = st.reshape(-1)
    if bits == 4:
        assert sf[0] == s[0, 0] and sf[1] == s[0, 1] and sf[2] == s[1, 0] and sf[32] == s[0, 2]
    else:
        assert sf[0] == s[0, 0] and sf[1] == s[1, 0] and (nsuper == 1 or sf[16] == s[0, 1])
    # every byte is placed exactly once; the padding rows are zero
    assert np.array_equal(np.sort(flat[flat != 0]), np.sort(wq.reshape(-1)[wq.reshape(-1) != 0]))
    w2, s2 = O.untile_weights(wt, st, bits, n)
    assert np.array_equal(w2, wq) and np.array_equal(s2.view(np.uint16), s.view(np.uint16))
    wpad, spad = O.untile_weights(wt, st, bits, rows)
    assert not wpad[n:].any() and not spad[n:].any()


# ---------------------------------------------------------------- gated tail: multiply(nn.silu(gate), up)
def _silu_both(g, u):
    y = np.concatenate([np.asarray(g, dtype=np.float16).reshape(1, -1), np.asarray(u, dtype=np.float16).reshape(1, -1)], axis=1)
    return O.epilogue(y, activation="silu_mul")[0], c_oracle.epilogue(y, activation="silu_mul")[0]


def test_silu_mul_known_answers_and_special_values():
    """Values the float16 operation sequence fixes by hand: silu(0) = 0; a large gate passes through
    (exp(-g) rounds to 0, 1 / 1 = 1); a gate of -20 gives exp(20) = inf in float16, 1 / inf = 0, -20 * 0 = -0;
    gate 1: e = f16(exp(-1)) = 0.36792, d = f16(1.36792) = 1.3682, s = f16(1 / 1.3682) = 0.73096, t = 0.73096."""
    g = np.array([0.0, 12.0, -20.0, 1.0, 1.0, -np.inf, np.inf, np.nan], dtype=np.float16)
    u = np.array([3.0, 0.5, 2.0, 1.0, -2.0, 1.0, 2.0, 1.0], dtype=np.float16)
    for got in _silu_both(g, u):
        assert got[0] == 0 and not np.signbit(got[0])
        assert got[1] == np.float16(6.0)
        assert got[2] == 0 and np.signbit(got[2])                     # -20 * (+0) = -0, times 2
        assert got[3].view(np.uint16) == np.float16(0.73096).view(np.uint16)
        assert got[4].view(np.uint16) == np.float16(-1.4619).view(np.uint16)
        assert np.isnan(got[5])                                       # -inf * 0
        assert got[6] == np.inf and np.isnan(got[7])


def test_silu_mul_both_restatements_agree_on_every_gate_value():
    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    for u in (1.0, -0.37, 23.5, 6.1e-5):
        a, b = _silu_both(halves, np.full(65536, u, dtype=np.float16))
        assert _bits_equal_nan_aware(a, b), u


def test_silu_mul_tracks_the_float64_closed_form():
    """g / (1 + exp(-g)) * u in float64 against the five-rounding float16 sequence: every result within
    6 float16 ulp (five roundings of half an ulp each, and an ulp is between 2^-11 and 2^-10 of its value, so
    errors carried across a power of two count double) -- a dropped term, a wrong sign or sigmoid in place of
    silu is off by orders of magnitude more."""
    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    # beyond |g| = 8 the sequence leaves the normal float16 range (1 / (1 + exp(9.7)) is subnormal, exp(11.1) overflows)
    # and below |g| = 2^-12 the product g * s is subnormal
    mag = np.abs(halves.astype(np.float64))
    g = halves[np.isfinite(halves) & (mag <= 8.0) & (mag >= 2.0 ** -12)]
    worst = 0.0
    for u in (1.0, -0.37, 23.5):
        got, _ = _silu_both(g, np.full(g.size, u, dtype=np.float16))
        g64 = g.astype(np.float64)
        exact = g64 / (1.0 + np.exp(-g64)) * np.float64(np.float16(u))
        ulp = np.maximum(np.spacing(np.abs(exact).astype(np.float16)).astype(np.float64), 2.0 ** -24)
        err = np.abs(got.astype(np.float64) - exact) / ulp
        worst = max(worst, float(err.max()))
    assert worst <= 6.0, worst


def test_silu_mul_every_step_against_exact_rationals():
    """Each of the four arithmetic steps (1 + e, 1 / d, g * s, t * u) rounded independently: exact fractions
    and a nearest-even search in the table of all float16 values; exp(-g) in float16 comes from `math.exp`
    (double precision) rounded by the same search."""
    import bisect
    import math
    from fractions import Fraction

    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    finite = halves[np.isfinite(halves) & ~((halves == 0) & np.signbit(halves))]
    table = finite[np.argsort(finite.astype(np.float64), kind="stable")]
    fracs = [Fraction(float(h)) for h in table]

    def nearest(fr):
        assert abs(fr) < 65520
        i = bisect.bisect_left(fracs, fr)
        cands = [j for j in (i - 1, i) if 0 <= j < len(fracs)]
        dist = [abs(fracs[j] - fr) for j in cands]
        if len(cands) == 2 and dist[0] == dist[1]:
            j = cands[0] if (int(table[cands[0]].view(np.uint16)) & 1) == 0 else cands[1]
        else:
            j = cands[int(np.argmin(dist))]
        return Fraction(float(table[j]))

    rng = np.random.default_rng(7)
    g = (rng.standard_normal(1500) * 3).astype(np.float16)
    u = (rng.standard_normal(1500) * 2).astype(np.float16)
    got_np, got_c = _silu_both(g, u)
    for i in range(g.size):
        gf, uf = Fraction(float(g[i])), Fraction(float(u[i]))
        e = nearest(Fraction(math.exp(-float(g[i]))))
        d = nearest(1 + e)
        s = nearest(1 / d)
        t = nearest(gf * s)
        want = nearest(t * uf)
        assert Fraction(float(got_np[i])) == want and Fraction(float(got_c[i])) == want, (g[i], u[i])


# ------------------------------------------------------------------ gelu (float16 operation sequence)
def test_gelu_python_and_c_oracles_agree_on_every_float16():
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    x = h[np.isfinite(h)].reshape(1, -1)
    a = O.epilogue(x, activation="gelu")
    b = c_oracle.epilogue(x, activation="gelu")
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


def test_gelu_closed_form_bound_on_every_float16():
    """x * Phi(x) in float64 against the float16 sequence x * (0.5 + erf(x * sqrt(0.5)) * 0.5).  Error budget of
    the sequence: the argument a = x * sqrt(0.5) carries a relative 2^-10 (constant and product rounded), which
    erf turns into at most (2/sqrt(pi)) |a| exp(-a^2) 2^-10 <= 0.484 * 2^-10; e adds 2^-12; halving is exact;
    c = 0.5 + b adds 2^-12: |c - Phi(x)| <= 0.5 (0.484 * 2^-10 + 2^-12) + 2^-12 < 2.5 * 2^-12, and the final
    product half a float16 ulp.  (For x < -1 the sum 0.5 + b cancels, so the sequence is far from x * Phi(x)
    in relative terms: that is a property of the legalized form, not of this restatement.)  A wrong constant,
    sign or a dropped term misses the bound by orders of magnitude."""
    import math

    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    x = h[np.isfinite(h)]
    got = O.gelu_f16(x).astype(np.float64)
    xf = x.astype(np.float64)
    exact = xf * 0.5 * (1.0 + np.vectorize(math.erf)(xf / math.sqrt(2.0)))
    ok = np.abs(exact) < 65504.0
    ulp = np.spacing(np.abs(exact[ok]).astype(np.float16)).astype(np.float64)
    bound = np.abs(xf[ok]) * 2.5 * 2.0 ** -12 + 0.5 * ulp + 2.0 ** -25
    assert np.all(np.abs(got[ok] - exact[ok]) <= bound)
    # the bound is not slack by orders of magnitude: some input uses more than half of it
    assert (np.abs(got[ok] - exact[ok]) / bound).max() > 0.5
    # mistakes the bound catches: sqrt(0.5) replaced by 0.5, the sign of erf, the missing 0.5 +
    for wrong in (xf * 0.5 * (1.0 + np.vectorize(math.erf)(xf * 0.5)),
                  xf * 0.5 * (1.0 - np.vectorize(math.erf)(xf / math.sqrt(2.0))),
                  xf * 0.5 * np.vectorize(math.erf)(xf / math.sqrt(2.0))):
        assert not np.all(np.abs(wrong[ok] - exact[ok]) <= bound)


def test_gelu_special_values_and_position_in_the_tail():
    f = np.float16
    x = np.array([[0.0, -0.0, 1.0, -1.0, 10.0, -10.0, np.inf, np.nan, 6e-8]], dtype=f)
    y = O.epilogue(x, activation="gelu")
    assert y[0, 0] == 0 and not np.signbit(y[0, 0]) and y[0, 1] == 0 and np.signbit(y[0, 1])
    assert y[0, 2] == f(0.8413) and y[0, 3] == f(-0.1587)
    assert y[0, 4] == f(10.0) and y[0, 5] == 0 and np.signbit(y[0, 5])  # c rounds to 1 / to 0
    assert np.isinf(y[0, 6]) and np.isnan(y[0, 7])
    assert y[0, 8] == f(6e-8) * f(0.5)
    # bias first, gelu second, residual last
    t = np.array([[0.5, -2.0]], dtype=f)
    bias = np.array([0.5, 1.0], dtype=f)
    res = np.array([[1.0, 1.0]], dtype=f)
    want = O.add_f16(O.gelu_f16(O.add_f16(t, bias.reshape(1, -1))), res)
    assert np.array_equal(O.epilogue(t, bias, "gelu", res), want)
    assert np.array_equal(c_oracle.epilogue(t, bias, "gelu", res), want)
