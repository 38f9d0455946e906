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
