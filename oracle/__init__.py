"""CPU oracle for the packed-int4 GEMM (test infrastructure, never shipped).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package, and only as the checker.
"""
from .qm_oracle import (  # noqa: F401
    build,
    compare,
    gemm_i4,
    gemm_i4_rows,
    gemm_i8,
    gemm_numpy,
    max_threads,
    OUT_BF16,
    OUT_F16,
    pack_i4,
    pack_numpy,
    quantize_pack,
    quantize_pack_numpy,
    scale_round16,
    scale_round16_numpy,
    unpack_i4,
    unpack_numpy,
)
