"""The Relax side of the boundary: pattern table, `relax.ext.mi355x` codegen hook and
the per-symbol C trampolines it emits.  Nothing here imports TVM at module import time;
`patterns()` and `register()` import it when called, `trampoline_source()` is plain text
generation and runs anywhere."""
from .codegen import CallSpec, register, trampoline_source  # noqa: F401
from .patterns import BACKEND, patterns  # noqa: F401
