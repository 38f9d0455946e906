"""CPU oracle for the weight-only-quantized dequantize + matmul path (NumPy).

TEST INFRASTRUCTURE ONLY.  Nothing that ships (the `relax_amd` package, the
C-ABI library) may import this module; only `tests/`, the smoke check and the
`cpu_baseline` leg of the benchmark use it, and only as the checker.

It restates, in closed form, what the reference's llvm-CPU path computes for the
canonical module

    Wd  = call_tir(decode_q{4,8}f16, (Wq, S))      # [N, K] float16
    y32 = matmul(x, permute_dims(Wd), out_dtype="float32")
    y   = astype(y32, "float16")

Reference semantics followed (file:line under the reference tree):

* integer unpack: `shift_right` on an unsigned operand is a logical shift,
  `bitwise_and` is a plain AND -- src/target/llvm/codegen_llvm.cc:1271-1285;
  uint -> int8 is an integer truncation and int/uint -> float16 is an exact
  SIToFP/UIToFP -- src/target/llvm/codegen_llvm.cc:820-852.
* float16 arithmetic in `decode` rounds to float16 after every operation
  (the result is stored to a float16 buffer in the unfused module).
* matmul: products `float32(a) * float32(b)` summed by a sequential float32
  reduction over ascending k starting from 0 --
  python/tvm/relax/transform/legalize_ops.py:203-264 and the golden TIR in
  tests/python/relax/test_transform_legalize_ops_index_linear_algebra.py:283-313.
* final cast float32 -> float16 is round-to-nearest-even (FPCast) --
  python/tvm/relax/transform/legalize_ops.py:157-162,
  src/target/llvm/codegen_llvm.cc:849-850.

* fused tail (composites with `relax.add` / `relax.nn.relu` behind the cast): each op is
  legalized to its own element-wise PrimFunc on float16 tensors
  (python/tvm/relax/transform/legalize_ops.py:632 and the binary-op table above it), so every
  add rounds once to float16; relu is max(t, 0) (python/tvm/topi/nn/elemwise.py:26-39),
  emitted as select(t > 0, t, 0) with an ordered compare
  (src/target/llvm/codegen_llvm.cc:1500-1504): -0 and NaN both give +0.

* gated tail (the gate+up projection of a Llama MLP followed by `multiply(nn.silu(gate), up)` on the two
  halves of the output): `relax.nn.silu` legalizes to `multiply(x, sigmoid(x))`
  (python/tvm/relax/transform/legalize_ops.py:506-510), `sigmoid` to `1 / (1 + exp(-x))` in the tensor's
  dtype (src/target/intrin_rule.cc:135-141) and `exp` to the llvm.exp intrinsic
  (src/target/llvm/intrin_rule_llvm.cc:41-42), which on a float16 operand is evaluated in float32
  (extend, expf, truncate).  Every float16 operation rounds once: e = f16(expf(-g)), d = f16(1 + e),
  s = f16(1 / d), t = f16(g * s), y = f16(t * u).  The one step that is not fixed by IEEE arithmetic is
  the last bit of expf (the host libm's); rounded to float16 it differs between correct
  implementations in about one operand in a few thousand.

Layout decisions frozen by this build (the reference holds no quantized path):
element k of a row lives in word k // per_word at bit offset
(k % per_word) * bits, least-significant field first.

Pinning (see tests/test_oracle.py): unpack against an independent pure-Python
bit walk over every field value and position; dequantize exhaustively against a
float64 closed form for all 16 x 65536 (q4) and 256 x 65536 (q8) operand pairs;
matmul against exact integer arithmetic, one-hot readback, a float64 bound and an
order-sensitive hand-computed case; the float16 add of the fused tail against exact
rational arithmetic (fractions) with an independent nearest-even search over all float16
values, and tie / overflow / signed-zero known answers; relu on the special values.
"""
from __future__ import annotations

import numpy as np

Q4_ZERO_POINT = 7
Q4_GROUP = 32
Q8_GROUP = 128


# ----------------------------------------------------------------------------
# packing (inverse of the decode index arithmetic; used to build test inputs)
# ----------------------------------------------------------------------------
def pack_q4(w: np.ndarray) -> np.ndarray:
    """[N, K] integers in 0..15 -> uint32 [N, K/8], field k%8 at bit (k%8)*4."""
    w = np.asarray(w)
    n, k = w.shape
    assert k % 8 == 0
    assert w.min(initial=0) >= 0 and w.max(initial=0) <= 15
    f = w.astype(np.uint32).reshape(n, k // 8, 8)
    out = np.zeros((n, k // 8), dtype=np.uint32)
    for i in range(8):
        out |= f[:, :, i] << np.uint32(4 * i)
    return out


def pack_q8(w: np.ndarray) -> np.ndarray:
    """[N, K] integers in -128..127 -> uint32 [N, K/4], byte k%4 at bit (k%4)*8."""
    w = np.asarray(w)
    n, k = w.shape
    assert k % 4 == 0
    assert w.min(initial=0) >= -128 and w.max(initial=0) <= 127
    f = (w.astype(np.int64) & 0xFF).astype(np.uint32).reshape(n, k // 4, 4)
    out = np.zeros((n, k // 4), dtype=np.uint32)
    for i in range(4):
        out |= f[:, :, i] << np.uint32(8 * i)
    return out


# ----------------------------------------------------------------------------
# decode: integer part
# ----------------------------------------------------------------------------
def unpack_q4(wq: np.ndarray) -> np.ndarray:
    """uint32 [N, K/8] -> uint8 [N, K]: (Wq[n, k//8] >> ((k%8)*4)) & 15."""
    wq = np.ascontiguousarray(wq, dtype=np.uint32)
    n, kw = wq.shape
    sh = (np.arange(8, dtype=np.uint32) * np.uint32(4))[None, None, :]
    return ((wq[:, :, None] >> sh) & np.uint32(15)).astype(np.uint8).reshape(n, kw * 8)


def unpack_q8(wq: np.ndarray) -> np.ndarray:
    """uint32 [N, K/4] -> int8 [N, K]: int8((Wq[n, k//4] >> ((k%4)*8)) & 255)."""
    wq = np.ascontiguousarray(wq, dtype=np.uint32)
    n, kw = wq.shape
    sh = (np.arange(4, dtype=np.uint32) * np.uint32(8))[None, None, :]
    b = ((wq[:, :, None] >> sh) & np.uint32(255)).astype(np.uint8)
    return b.view(np.int8).reshape(n, kw * 4)  # two's-complement truncation


# ----------------------------------------------------------------------------
# decode: float16 part (one rounding per float16 operation)
# ----------------------------------------------------------------------------
def dequant_q4f16(wq, s, group: int = Q4_GROUP, zero_point: int = Q4_ZERO_POINT) -> np.ndarray:
    """Wd[n,k] = (f16(w) - f16(zp)) * S[n, k//group], each op rounded to f16."""
    w = unpack_q4(wq)
    n, k = w.shape
    s = np.asarray(s, dtype=np.float16)
    assert s.shape == (n, k // group) and k % group == 0
    centred = w.astype(np.float16) - np.float16(zero_point)  # exact, |.| <= 15
    with np.errstate(all="ignore"):
        return centred * np.repeat(s, group, axis=1)  # float16 multiply: single RNE


def dequant_q8f16(wq, s, group: int = Q8_GROUP) -> np.ndarray:
    """Wd[n,k] = f16(int8 field) * S[n, k//group]."""
    w = unpack_q8(wq)
    n, k = w.shape
    s = np.asarray(s, dtype=np.float16)
    assert s.shape == (n, k // group) and k % group == 0
    with np.errstate(all="ignore"):
        return w.astype(np.float16) * np.repeat(s, group, axis=1)


def dequant(wq, s, bits: int, group: int) -> np.ndarray:
    if bits == 4:
        return dequant_q4f16(wq, s, group)
    if bits == 8:
        return dequant_q8f16(wq, s, group)
    raise ValueError(f"bits must be 4 or 8, got {bits}")


# ----------------------------------------------------------------------------
# matmul + cast
# ----------------------------------------------------------------------------
def matmul_f32acc(x: np.ndarray, wd: np.ndarray) -> np.ndarray:
    """y32[m,n] = sum_k f32(x[m,k]) * f32(Wd[n,k]); float32, k ascending, init 0.

    Vectorised over (m, n); the k loop is explicit so every output element sees
    exactly the reference's sequence of float32 additions.
    """
    x32 = np.asarray(x, dtype=np.float16).astype(np.float32)
    w32 = np.asarray(wd, dtype=np.float16).astype(np.float32)
    m, k = x32.shape
    n, k2 = w32.shape
    assert k == k2
    acc = np.zeros((m, n), dtype=np.float32)
    wt = np.ascontiguousarray(w32.T)  # [K, N]
    with np.errstate(all="ignore"):
        for kk in range(k):
            acc += x32[:, kk, None] * wt[kk][None, :]  # product exact in f32, one f32 add
    return acc


def cast_f16(y32: np.ndarray) -> np.ndarray:
    with np.errstate(all="ignore"):
        return np.asarray(y32, dtype=np.float32).astype(np.float16)


def wq_matmul(x, wq, s, bits: int, group: int) -> np.ndarray:
    """The whole path: y = f16( x @ dequant(Wq, S)^T ) with float32 accumulation."""
    return cast_f16(matmul_f32acc(x, dequant(wq, s, bits, group)))


# ----------------------------------------------------------------------------
# synthetic inputs of the benchmark's distributions
# ----------------------------------------------------------------------------
def add_f16(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """IEEE binary16 addition, one rounding (broadcasting like `relax.add`).

    The exact sum of two float16 values is computed in float64 (exact: both operands are
    multiples of 2^-24 below 2^16, so the sum has at most 41 significant bits) and rounded
    once to float16."""
    a = np.asarray(a, dtype=np.float16)
    b = np.asarray(b, dtype=np.float16)
    with np.errstate(over="ignore", invalid="ignore"):
        return (a.astype(np.float64) + b.astype(np.float64)).astype(np.float16)


def relu_f16(t: np.ndarray) -> np.ndarray:
    """select(t > 0, t, 0): negative values, -0 and NaN become +0."""
    t = np.asarray(t, dtype=np.float16)
    with np.errstate(invalid="ignore"):
        return np.where(t > np.float16(0), t, np.float16(0)).astype(np.float16)


def silu_mul_f16(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """multiply(nn.silu(gate), up) on float16 tensors, every operation rounded once to float16:
    e = f16(expf(-g)); d = f16(1 + e); s = f16(1 / d); t = f16(g * s); y = f16(t * u).
    expf is taken as the correctly rounded float32 exponential (float64 exp rounded to float32: what
    glibc's expf returns in all but astronomically rare cases); sums and products of two float16 values
    are exact in float64 before their single rounding."""
    g = np.asarray(gate, dtype=np.float16)
    u = np.asarray(up, dtype=np.float16)
    with np.errstate(over="ignore", invalid="ignore", divide="ignore", under="ignore"):
        e = np.exp(-g.astype(np.float64)).astype(np.float32).astype(np.float16)
        d = (np.float64(1) + e.astype(np.float64)).astype(np.float16)
        # 1 / d in float32 is correctly rounded and 24 >= 2 * 11 + 2 bits make the second rounding innocuous
        s = (np.float32(1) / d.astype(np.float32)).astype(np.float16)
        t = (g.astype(np.float64) * s.astype(np.float64)).astype(np.float16)
        return (t.astype(np.float64) * u.astype(np.float64)).astype(np.float16)


def gelu_f16(t: np.ndarray) -> np.ndarray:
    """nn.gelu on a float16 tensor as its legalized form x * (0.5 + erf(x * sqrt(0.5)) * 0.5)
    (python/tvm/relax/transform/legalize_ops.py:495-503) runs on float16, one rounding per operation and the
    constants rounded to float16 first: a = f16(x * f16(sqrt(0.5))); e = f16(erff(a)); b = f16(e * 0.5);
    c = f16(0.5 + b); y = f16(x * c).  erff is taken as the float64 erf rounded to float32.  The reference's
    CPU path cannot lower a float16 erf (src/target/intrin_rule.h:39-48), so this sequence has no reference
    output to be compared with: it is pinned in closed form against x * Phi(x)."""
    import math

    x = np.asarray(t, dtype=np.float16)
    c0 = np.float16(0.5 ** 0.5)
    with np.errstate(over="ignore", invalid="ignore", under="ignore"):
        a = (x.astype(np.float64) * np.float64(c0)).astype(np.float16)
        erf = np.vectorize(math.erf, otypes=[np.float64])
        e = erf(a.astype(np.float64)).astype(np.float32).astype(np.float16)
        b = (e.astype(np.float64) * 0.5).astype(np.float16)
        c = (np.float64(0.5) + b.astype(np.float64)).astype(np.float16)
        return (x.astype(np.float64) * c.astype(np.float64)).astype(np.float16)


def gated_epilogue(y: np.ndarray) -> np.ndarray:
    """y [M, N] = f16(accumulator) of a fused gate+up projection -> [M, N/2]:
    multiply(nn.silu(y[:, :N/2]), y[:, N/2:])."""
    y = np.asarray(y, dtype=np.float16)
    if y.ndim != 2 or y.shape[1] % 2 != 0:
        raise ValueError("the gated tail needs an even number of output columns")
    half = y.shape[1] // 2
    return silu_mul_f16(y[:, :half], y[:, half:])


def epilogue(y: np.ndarray, bias=None, activation: str | None = None, residual=None) -> np.ndarray:
    """The fused tail of a composite applied to y = f16(accumulator):
    + bias[N], then relu or gelu, then + residual[M,N]; every step absent or float16 ops rounded one by one."""
    t = np.asarray(y, dtype=np.float16)
    if activation == "silu_mul":
        if bias is not None or residual is not None:
            raise ValueError("the gated tail takes no bias or residual")
        return gated_epilogue(t)
    if bias is not None:
        t = add_f16(t, np.asarray(bias, dtype=np.float16).reshape(1, -1))
    if activation in ("relu", "relax.nn.relu"):
        t = relu_f16(t)
    elif activation in ("gelu", "relax.nn.gelu"):
        t = gelu_f16(t)
    elif activation not in (None, "none"):
        raise ValueError(f"unsupported activation {activation!r}")
    if residual is not None:
        t = add_f16(t, residual)
    return t


def wq_matmul_fused(x, wq, s, bits: int, group: int, bias=None, activation: str | None = None,
                    residual=None) -> np.ndarray:
    """y = epilogue(f16(x @ dequant(Wq, S)^T))."""
    return epilogue(wq_matmul(x, wq, s, bits, group), bias, activation, residual)


# ---------------------------------------------------------------- tile-major weight layout
# No counterpart in the reference (its weights stay row-major): the definition below is this
# build's own, restated with explicit loops so that the device transform has something
# independent to be compared with.  Chunk = 16 bytes of a weight row, super step = 8 chunks,
# tile = 16 rows; S = super steps per row.
#   weights: chunk (row t*16 + col, index s*8 + kq*2 + d) -> 16 bytes at ((t*S + s)*2 + d)*1024 + (kq*16 + col)*16
#   scales : int4 / group 32 -> float16 at (((t*S + s)*64 + kq*16 + col)*2 + e)*2 for group s*8 + kq*2 + e
#            int8 / group 128 -> float16 at ((t*S + s)*16 + col)*2 for group s
def tile_weights(wq: np.ndarray, s: np.ndarray, bits: int):
    """Canonical (wq [N, K*bits/32] uint32, scales [N, K/group] float16) -> tile-major arrays of the same
    shapes with N rounded up to 16 rows (bytes in tile-major order; rows past N are zero)."""
    n, words = wq.shape
    nsuper = words * 4 // 128
    assert words * 4 % 128 == 0 and s.shape == (n, nsuper * (8 if bits == 4 else 1))
    tiles = (n + 15) // 16
    wt = np.zeros(tiles * nsuper * 2 * 64 * 4, np.uint32)
    st = np.zeros(tiles * nsuper * (128 if bits == 4 else 16), np.float16)
    for row in range(n):
        t, col = divmod(row, 16)
        for chunk in range(nsuper * 8):
            sstep, r = divmod(chunk, 8)
            kq, d = divmod(r, 2)
            dst = (((t * nsuper + sstep) * 2 + d) * 64 + kq * 16 + col) * 4
            wt[dst:dst + 4] = wq[row, chunk * 4:chunk * 4 + 4]
            if bits == 4:
                st[((t * nsuper + sstep) * 64 + kq * 16 + col) * 2 + d] = s[row, chunk]
        if bits == 8:
            for sstep in range(nsuper):
                st[(t * nsuper + sstep) * 16 + col] = s[row, sstep]
    return wt.reshape(tiles * 16, words), st.reshape(tiles * 16, s.shape[1])


def untile_weights(wt: np.ndarray, st: np.ndarray, bits: int, n: int):
    """Inverse of tile_weights (vectorized independently of it: reshape / transpose)."""
    rows, words = wt.shape
    tiles, nsuper = rows // 16, words * 4 // 128
    w = wt.reshape(tiles, nsuper, 2, 4, 16, 4).transpose(0, 4, 1, 3, 2, 5).reshape(rows, words)  # [t,s,d,kq,col,4] -> [t,col,s,kq,d,4]
    if bits == 4:
        sc = st.reshape(tiles, nsuper, 4, 16, 2).transpose(0, 3, 1, 2, 4).reshape(rows, nsuper * 8)  # [t,s,kq,col,e] -> [t,col,s,kq,e]
    else:
        sc = st.reshape(tiles, nsuper, 16).transpose(0, 2, 1).reshape(rows, nsuper)
    return np.ascontiguousarray(w[:n]), np.ascontiguousarray(sc[:n])


def make_case(seed: int, m: int, n: int, k: int, bits: int, group: int | None = None):
    """x ~ N(0,1) f16; q4: w ~ U{0..15}, S ~ U(0.005,0.02); q8: w ~ U{-127..127}, S ~ U(0.002,0.01)."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k), dtype=np.float32).astype(np.float16)
    if bits == 4:
        group = group or Q4_GROUP
        w = rng.integers(0, 16, size=(n, k), dtype=np.int64)
        wq = pack_q4(w)
        s = rng.uniform(0.005, 0.02, size=(n, k // group)).astype(np.float16)
    elif bits == 8:
        group = group or Q8_GROUP
        w = rng.integers(-127, 128, size=(n, k), dtype=np.int64)
        wq = pack_q8(w)
        s = rng.uniform(0.002, 0.01, size=(n, k // group)).astype(np.float16)
    else:
        raise ValueError(bits)
    return x, wq, s, group
