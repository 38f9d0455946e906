"""Writes the golden fixtures (inputs + oracle outputs) used by the CPU and GPU tests.

The reference holds no vectors for a quantized matmul (it has no such operator), so the
fixtures are outputs of the pinned CPU oracle on seeded inputs; they freeze the layout
(least-significant field first) and the rounding sequence.  Run from the repo root:

    python tests/golden/make_golden.py            (--fused-only / --tiled-only / --tails-only: just those fixtures)
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import wq_oracle as O  # noqa: E402

CASES = [  # name, seed, M, N, K, bits, group
    ("q4f16_m3_n48_k96", 11, 3, 48, 96, 4, 32),
    ("q4f16_m1_n64_k352", 12, 1, 64, 352, 4, 32),
    ("q4f16_m70_n40_k128", 13, 70, 40, 128, 4, 32),
    ("q8f16_m5_n40_k256", 14, 5, 40, 256, 8, 128),
    ("q8f16_m66_n24_k384", 15, 66, 24, 384, 8, 128),
]

FUSED_CASES = [  # name, seed, M, N, K, bits, group, bias?, activation, residual?
    ("fused_q4f16_m4_n48_k128_bias_relu_res", 21, 4, 48, 128, 4, 32, True, "relu", True),
    ("fused_q4f16_m1_n80_k256_res", 22, 1, 80, 256, 4, 32, False, None, True),
    ("fused_q8f16_m70_n24_k256_bias", 23, 70, 24, 256, 8, 128, True, None, False),
]


TAIL_CASES = [  # name, seed, M, N, K, bits, group, bias?, activation: the tails with a float32 transcendental inside
    ("tail_q4f16_m6_n64_k256_bias_gelu", 41, 6, 64, 256, 4, 32, True, "gelu"),
    ("tail_q8f16_m9_n48_k256_silu_mul", 42, 9, 48, 256, 8, 128, False, "silu_mul"),
]


TILED_CASES = [  # name, seed, N, K, bits: the tile-major layout frozen as data (it is a storage format)
    ("tiled_q4f16_n37_k512", 31, 37, 512, 4),
    ("tiled_q8f16_n50_k384", 32, 50, 384, 8),
]


def fused_operands(seed, m, n, with_bias, with_residual):
    """bias ~ N(0, 0.5), residual ~ N(0, 1), float16, from their own seeded stream."""
    rng = np.random.default_rng(1000 + seed)
    bias = (0.5 * rng.standard_normal(n, dtype=np.float32)).astype(np.float16) if with_bias else None
    res = rng.standard_normal((m, n), dtype=np.float32).astype(np.float16) if with_residual else None
    return bias, res


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    for name, seed, n, k, bits in TILED_CASES:
        _, wq, s, g = O.make_case(seed, 1, n, k, bits)
        wt, st = O.tile_weights(wq, s, bits)
        np.savez_compressed(os.path.join(here, name + ".npz"), wq=wq, scales=s, wq_tiled=wt, scales_tiled=st,
                            bits=np.int32(bits), group=np.int32(g))
        print(name, wt.shape, st.shape)
    if "--tiled-only" in sys.argv:
        sys.exit(0)
    for name, seed, m, n, k, bits, group, wb, act in TAIL_CASES:
        x, wq, s, g = O.make_case(seed, m, n, k, bits, group)
        bias, _ = fused_operands(seed, m, n, wb, False)
        y = O.wq_matmul_fused(x, wq, s, bits, g, bias, act, None)
        extra = {} if bias is None else {"bias": bias}
        np.savez_compressed(os.path.join(here, name + ".npz"), x=x, wq=wq, scales=s, y=y,
                            y_plain=O.wq_matmul(x, wq, s, bits, g), bits=np.int32(bits), group=np.int32(g),
                            activation=np.array(act), **extra)
        print(name, y.shape, float(np.abs(y).max()))
    if "--tails-only" in sys.argv:
        sys.exit(0)
    for name, seed, m, n, k, bits, group, wb, act, wr in FUSED_CASES:
        x, wq, s, g = O.make_case(seed, m, n, k, bits, group)
        bias, res = fused_operands(seed, m, n, wb, wr)
        y = O.wq_matmul_fused(x, wq, s, bits, g, bias, act, res)
        extra = {}
        if bias is not None:
            extra["bias"] = bias
        if res is not None:
            extra["residual"] = res
        np.savez_compressed(os.path.join(here, name + ".npz"), x=x, wq=wq, scales=s, y=y,
                            y_plain=O.wq_matmul(x, wq, s, bits, g), bits=np.int32(bits), group=np.int32(g),
                            activation=np.array(act or "none"), **extra)
        print(name, y.shape, float(np.abs(y).max()))
    if "--fused-only" in sys.argv:
        sys.exit(0)
    for name, seed, m, n, k, bits, group in CASES:
        x, wq, s, g = O.make_case(seed, m, n, k, bits, group)
        wd = O.dequant(wq, s, bits, g)
        y = O.wq_matmul(x, wq, s, bits, g)
        np.savez_compressed(os.path.join(here, name + ".npz"), x=x, wq=wq, scales=s, wd=wd, y=y,
                            bits=np.int32(bits), group=np.int32(g))
        print(name, y.shape, float(np.abs(y).max()))
