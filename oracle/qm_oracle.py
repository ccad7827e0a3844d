"""ctypes front-end of ``libqm_oracle.so`` plus a numpy restatement of the same path.

TEST INFRASTRUCTURE ONLY: the shipped package never imports this module.

Two independent statements of the reference's CPU path are kept here so that each
can check the other:

* the C library (``qm_oracle.c``), which follows ``cpu_gemm_int8``
  (kernel.cu:291-306), ``unpack_int4_matrix`` (kernel.cu:387-408) and ``pack_b``
  (test.py:6-15) loop for loop;
* ``gemm_numpy`` / ``pack_numpy`` / ``unpack_numpy``, vectorised numpy written
  from the same definitions (int64 matmul, bit masks).

The reference ships no golden vectors for this path (test.py:22-23 draws unseeded
inputs), so both are pinned by closed forms in ``tests/test_oracle_pins.py``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libqm_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``qm_oracle.c`` with gcc (``make -C oracle``); returns the .so path."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, stdout=subprocess.DEVNULL)
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    u8p, i8p, i32p = ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p
    ci = ctypes.c_int
    lib.qm_oracle_unpack_i4.argtypes = [u8p, i8p, ci, ci]
    lib.qm_oracle_unpack_i4.restype = None
    lib.qm_oracle_pack_i4.argtypes = [i8p, u8p, ci, ci]
    lib.qm_oracle_pack_i4.restype = None
    lib.qm_oracle_gemm_i8.argtypes = [i8p, i8p, i32p, ci, ci, ci]
    lib.qm_oracle_gemm_i8.restype = None
    lib.qm_oracle_gemm_i8_mt.argtypes = [i8p, i8p, i32p, ci, ci, ci, ci]
    lib.qm_oracle_gemm_i8_mt.restype = ci
    lib.qm_oracle_gemm_i4.argtypes = [u8p, u8p, i32p, ci, ci, ci, ci]
    lib.qm_oracle_gemm_i4.restype = ci
    lib.qm_oracle_gemm_i4_rows.argtypes = [u8p, u8p, i32p, i32p, ci, ci, ci, ci, ci]
    lib.qm_oracle_gemm_i4_rows.restype = ci
    lib.qm_oracle_compare.argtypes = [i32p, i32p, ctypes.c_longlong]
    lib.qm_oracle_compare.restype = ctypes.c_longlong
    lib.qm_oracle_scale_round16.argtypes = [i32p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ci, ci, ci]
    lib.qm_oracle_scale_round16.restype = ci
    lib.qm_oracle_quantize_pack.argtypes = [ctypes.c_void_p, u8p, ctypes.c_void_p, ci, ci]
    lib.qm_oracle_quantize_pack.restype = ci
    lib.qm_oracle_max_threads.argtypes = []
    lib.qm_oracle_max_threads.restype = ci
    _lib = lib
    return lib


def _ptr(a: np.ndarray):
    return ctypes.c_void_p(a.ctypes.data)


def _as_bytes(a) -> np.ndarray:
    """Packed operands may arrive as int8 (what pack_b yields, test.py:14) or uint8."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.int8:
        a = a.view(np.uint8)
    if a.dtype != np.uint8:
        raise TypeError(f"packed int4 data must be int8/uint8, got {a.dtype}")
    return a


def max_threads() -> int:
    return int(_load().qm_oracle_max_threads())


def unpack_i4(packed) -> np.ndarray:
    """[rows, K/2] bytes -> [rows, K] int8 (kernel.cu:389-408)."""
    p = _as_bytes(packed)
    rows, half = p.shape
    out = np.empty((rows, 2 * half), dtype=np.int8)
    _load().qm_oracle_unpack_i4(_ptr(p), _ptr(out), rows, 2 * half)
    return out


def pack_i4(values) -> np.ndarray:
    """[rows, K] int8 holding int4 values -> [rows, K/2] uint8 (test.py:6-15)."""
    v = np.ascontiguousarray(values, dtype=np.int8)
    rows, K = v.shape
    if K % 2:
        raise ValueError("K must be even")
    out = np.empty((rows, K // 2), dtype=np.uint8)
    _load().qm_oracle_pack_i4(_ptr(v), _ptr(out), rows, K)
    return out


def gemm_i8(A, B, threads: int = 1) -> np.ndarray:
    """Unpacked int8 operands: C = A @ B.T in int32 (kernel.cu:291-306)."""
    A = np.ascontiguousarray(A, dtype=np.int8)
    B = np.ascontiguousarray(B, dtype=np.int8)
    M, K = A.shape
    N, K2 = B.shape
    if K != K2:
        raise ValueError("A and B disagree on K")
    C = np.empty((M, N), dtype=np.int32)
    if threads == 1:
        _load().qm_oracle_gemm_i8(_ptr(A), _ptr(B), _ptr(C), M, N, K)
    else:
        _load().qm_oracle_gemm_i8_mt(_ptr(A), _ptr(B), _ptr(C), M, N, K, threads)
    return C


def gemm_i4(A_packed, B_packed, threads: int = 0) -> np.ndarray:
    """Packed operands: unpack then multiply, as the reference's harness does
    (kernel.cu:447-448,505).  threads=1 is the reference's single-thread loop."""
    Ap, Bp = _as_bytes(A_packed), _as_bytes(B_packed)
    M, half = Ap.shape
    N, half2 = Bp.shape
    if half != half2:
        raise ValueError("A and B disagree on K")
    C = np.empty((M, N), dtype=np.int32)
    rc = _load().qm_oracle_gemm_i4(_ptr(Ap), _ptr(Bp), _ptr(C), M, N, 2 * half, threads)
    if rc < 0:
        raise RuntimeError("qm_oracle_gemm_i4 rejected its arguments")
    return C


def gemm_i4_rows(A_packed, B_packed, rows, threads: int = 0) -> np.ndarray:
    """Selected rows of C only (for spot-checking products too large to redo in full)."""
    Ap, Bp = _as_bytes(A_packed), _as_bytes(B_packed)
    M, half = Ap.shape
    N, _ = Bp.shape
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    C = np.empty((len(rows), N), dtype=np.int32)
    rc = _load().qm_oracle_gemm_i4_rows(_ptr(Ap), _ptr(Bp), _ptr(C), _ptr(rows), len(rows), M, N, 2 * half, threads)
    if rc < 0:
        raise RuntimeError("qm_oracle_gemm_i4_rows rejected its arguments")
    return C


def compare(got, want) -> int:
    """-1 when identical, else the flat index of the first mismatch (kernel.cu:308-319)."""
    g = np.ascontiguousarray(got, dtype=np.int32)
    w = np.ascontiguousarray(want, dtype=np.int32)
    if g.shape != w.shape:
        raise ValueError("shape mismatch")
    return int(_load().qm_oracle_compare(_ptr(g), _ptr(w), g.size))


OUT_F16, OUT_BF16 = 1, 2


def quantize_pack(x):
    """Per-row symmetric int4 quantisation fused with pack_b's packing (no counterpart in the
    reference).  ``x``: [rows, k] float32 (widen fp16 / bf16 first: exact).  Returns (packed
    uint8 [rows, k/2], scales float32 [rows]) with scale = amax / 7 and
    q = clamp(rint(x * (7 / amax)), -7, 7)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, k = x.shape
    packed = np.empty((rows, k // 2), dtype=np.uint8)
    scales = np.empty(rows, dtype=np.float32)
    rc = _load().qm_oracle_quantize_pack(x.ctypes.data, _ptr(packed), scales.ctypes.data, rows, k)
    if rc < 0:
        raise RuntimeError("qm_oracle_quantize_pack rejected its arguments")
    return packed, scales


def quantize_pack_numpy(x):
    """The same in numpy (float32 throughout, np.rint = round half to even)."""
    x = np.asarray(x, dtype=np.float32)
    amax = np.abs(x).max(axis=1) if x.shape[1] else np.zeros(x.shape[0], np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(amax > 0, np.float32(7.0) / amax, np.float32(0)).astype(np.float32)
    q = np.clip(np.rint((x * inv[:, None]).astype(np.float32)), -7, 7).astype(np.int8)
    return pack_numpy(q), (amax / np.float32(7.0)).astype(np.float32)


def scale_round16(C, row_scale, col_scale, out: int) -> np.ndarray:
    """uint16 bit patterns of round16(((float32)C * row_scale[m]) * col_scale[n]); ``out`` is
    OUT_F16 or OUT_BF16; a scale of None stands for all ones.  (No counterpart in the reference.)"""
    C = np.ascontiguousarray(C, dtype=np.int32)
    M, N = C.shape
    rs = None if row_scale is None else np.ascontiguousarray(row_scale, dtype=np.float32)
    cs = None if col_scale is None else np.ascontiguousarray(col_scale, dtype=np.float32)
    if (rs is not None and rs.shape != (M,)) or (cs is not None and cs.shape != (N,)):
        raise ValueError("scale shapes")
    D = np.empty((M, N), dtype=np.uint16)
    rc = _load().qm_oracle_scale_round16(_ptr(C), None if rs is None else rs.ctypes.data, None if cs is None else cs.ctypes.data,
                                         D.ctypes.data, M, N, out)
    if rc < 0:
        raise RuntimeError("qm_oracle_scale_round16 rejected its arguments")
    return D


def scale_round16_numpy(C, row_scale, col_scale, out: int) -> np.ndarray:
    """The same in numpy: float32 products in the same order, numpy's own float16 cast, and
    bfloat16 by the add-0x7FFF-plus-lsb rule on the bit pattern."""
    y = np.asarray(C, dtype=np.int32).astype(np.float32)
    if row_scale is not None:
        y = (y * np.asarray(row_scale, dtype=np.float32)[:, None]).astype(np.float32)
    if col_scale is not None:
        y = (y * np.asarray(col_scale, dtype=np.float32)[None, :]).astype(np.float32)
    if out == OUT_F16:
        with np.errstate(over="ignore"):
            return y.astype(np.float16).view(np.uint16)
    u = y.view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)


# ---------------------------------------------------------------- numpy restatement
def unpack_numpy(packed) -> np.ndarray:
    p = _as_bytes(packed)
    lo = (p & 0x0F).astype(np.int16)
    hi = (p >> 4).astype(np.int16)
    lo = np.where(lo > 7, lo - 16, lo)
    hi = np.where(hi > 7, hi - 16, hi)
    out = np.empty((p.shape[0], p.shape[1] * 2), dtype=np.int8)
    out[:, 0::2] = lo
    out[:, 1::2] = hi
    return out


def pack_numpy(values) -> np.ndarray:
    v = np.asarray(values, dtype=np.int8)
    flat = v.reshape(-1)
    flat = np.where(flat < 0, flat + 16, flat).astype(np.int8)
    packed = flat[0::2] | (flat[1::2] << 4).astype(np.int8)
    return packed.reshape(v.shape[0], v.shape[1] // 2).view(np.uint8)


def gemm_numpy(A_packed, B_packed) -> np.ndarray:
    A = unpack_numpy(A_packed).astype(np.int64)
    B = unpack_numpy(B_packed).astype(np.int64)
    return (A @ B.T).astype(np.int32)
