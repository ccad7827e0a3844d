"""quadmul_amd: packed-int4 GEMM for MI355X (gfx950), host-side interface.

Two ways in, both ending in the same C ABI (``include/qm_abi.h``,
``quadmul_amd/lib/libqm_hip.so``):

* the PyTorch-ROCm extension module ``quadmul`` (repo root), the drop-in for the
  reference's module of the same name: ``quadmul.gemm(a, b, c, m, n, k)``
  (extension.cpp:8-29, call site test.py:40);
* this package, which binds the C ABI with ctypes and takes torch tensors only to
  borrow their device pointers and the current stream.

There is no CPU or eager fallback for the GEMM: if the HIP library has not been
built, every call raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional

import torch

__all__ = [
    "QuadmulError", "library", "library_path", "gemm", "gemm_cfg", "gemm_static", "gemm_scaled", "pack_int4", "unpack_int4",
    "config_has_scaled", "quantize_pack",
    "num_configs", "config_name", "config_names", "config_id", "select_config", "select_config_ex", "config_supports",
    "CFG_AUTO", "version", "init",
]

_PKG = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_PKG, "lib", "libqm_hip.so")
_lib: Optional[ctypes.CDLL] = None

CFG_AUTO = -1
#: every symbol include/qm_abi.h declares
ABI_SYMBOLS = (
    "qm_gemm_i4", "qm_gemm_i4_cfg", "qm_gemm_i4_scaled", "qm_gemm_i4_scaled_cfg", "qm_config_has_scaled",
    "qm_gemm_i4_ws", "qm_gemm_i4_static", "qm_gemm_i4_scaled_ws", "qm_gemm_workspace_bytes", "qm_quantize_pack_i4", "qm_select_config", "qm_select_config_ex", "qm_num_configs", "qm_config_name",
    "qm_config_supports", "qm_pack_i4", "qm_unpack_i4", "qm_status_string", "qm_last_hip_error", "qm_version", "qm_init",
    "qm_debug_set_operand_limit",
)


class QuadmulError(RuntimeError):
    """A non-zero status from libqm_hip.so."""


def library_path() -> str:
    return _LIB_PATH


def library() -> ctypes.CDLL:
    """The loaded C-ABI library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise QuadmulError(
            f"{_LIB_PATH} is missing: build it with `python -m quadmul_amd.build` "
            "(there is no fallback path for the int4 GEMM)")
    lib = ctypes.CDLL(_LIB_PATH)
    vp, ci = ctypes.c_void_p, ctypes.c_int
    lib.qm_gemm_i4.argtypes = [vp, vp, vp, ci, ci, ci, vp]
    lib.qm_gemm_i4.restype = ci
    lib.qm_gemm_i4_cfg.argtypes = [vp, vp, vp, ci, ci, ci, vp, ci]
    lib.qm_gemm_i4_cfg.restype = ci
    lib.qm_gemm_i4_scaled.argtypes = [vp, vp, vp, ci, ci, ci, vp, vp, ci, vp]
    lib.qm_gemm_i4_scaled.restype = ci
    lib.qm_gemm_i4_scaled_cfg.argtypes = [vp, vp, vp, ci, ci, ci, vp, vp, ci, vp, ci]
    lib.qm_gemm_i4_scaled_cfg.restype = ci
    lib.qm_gemm_i4_ws.argtypes = [vp, vp, vp, ci, ci, ci, vp, ci, vp, ctypes.c_size_t]
    lib.qm_gemm_i4_ws.restype = ci
    lib.qm_gemm_i4_static.argtypes = [vp, vp, vp, ci, ci, ci, vp]
    lib.qm_gemm_i4_static.restype = ci
    lib.qm_gemm_i4_scaled_ws.argtypes = [vp, vp, vp, ci, ci, ci, vp, vp, ci, vp, ci, vp, ctypes.c_size_t]
    lib.qm_gemm_i4_scaled_ws.restype = ci
    lib.qm_gemm_workspace_bytes.argtypes = [ci, ci, ci, ci, ci, ci]
    lib.qm_gemm_workspace_bytes.restype = ctypes.c_size_t
    lib.qm_config_has_scaled.argtypes = [ci]
    lib.qm_config_has_scaled.restype = ci
    lib.qm_quantize_pack_i4.argtypes = [vp, ci, vp, vp, ci, ci, vp]
    lib.qm_quantize_pack_i4.restype = ci
    lib.qm_select_config.argtypes = [ci, ci, ci, ci]
    lib.qm_select_config.restype = ci
    lib.qm_select_config_ex.argtypes = [ci, ci, ci, ci, ci, ci]
    lib.qm_select_config_ex.restype = ci
    lib.qm_num_configs.argtypes = []
    lib.qm_num_configs.restype = ci
    lib.qm_config_name.argtypes = [ci]
    lib.qm_config_name.restype = ctypes.c_char_p
    lib.qm_config_supports.argtypes = [ci, ci, ci, ci, ci]
    lib.qm_config_supports.restype = ci
    lib.qm_pack_i4.argtypes = [vp, vp, ci, ci, vp]
    lib.qm_pack_i4.restype = ci
    lib.qm_unpack_i4.argtypes = [vp, vp, ci, ci, vp]
    lib.qm_unpack_i4.restype = ci
    lib.qm_status_string.argtypes = [ci]
    lib.qm_status_string.restype = ctypes.c_char_p
    lib.qm_last_hip_error.argtypes = []
    lib.qm_last_hip_error.restype = ci
    lib.qm_init.argtypes = []
    lib.qm_init.restype = ci
    lib.qm_version.argtypes = []
    lib.qm_version.restype = ctypes.c_char_p
    lib.qm_debug_set_operand_limit.argtypes = [ctypes.c_longlong]
    lib.qm_debug_set_operand_limit.restype = ctypes.c_longlong
    _lib = lib
    return lib


def _check(status: int, what: str) -> None:
    if status == 0:
        return
    lib = library()
    msg = lib.qm_status_string(status).decode()
    if status == -4:
        msg += f" (hipError_t {lib.qm_last_hip_error()})"
    raise QuadmulError(f"{what}: {msg}")


def _stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _is_byte(t: torch.Tensor) -> bool:
    return t.dtype in (torch.int8, torch.uint8)


def _check_operands(a, b, c, m, n, k, c_dtypes=(torch.int32,)) -> None:
    # The checks the reference left commented out (extension.cpp:11-15).
    if not (a.is_cuda and b.is_cuda and c.is_cuda):
        raise QuadmulError("gemm: a, b and c must be GPU tensors")
    if not (a.device == b.device == c.device):
        raise QuadmulError("gemm: all tensors must be on the same device")
    if not (_is_byte(a) and _is_byte(b)):
        raise QuadmulError("gemm: a and b must be int8 or uint8 (packed int4)")
    if c.dtype not in c_dtypes:
        raise QuadmulError("gemm: c must be " + " or ".join(str(d).replace("torch.", "") for d in c_dtypes))
    if not (a.is_contiguous() and b.is_contiguous() and c.is_contiguous()):
        raise QuadmulError("gemm: all tensors must be contiguous")
    if m < 0 or n < 0 or k < 0 or k % 2:
        raise QuadmulError("gemm: m, n, k must be >= 0 and k even")
    if a.numel() != m * (k // 2) or b.numel() != n * (k // 2) or c.numel() != m * n:
        raise QuadmulError("gemm: tensor sizes do not match m, n, k")


def _ptr_align(*tensors) -> int:
    x = 0
    for t in tensors:
        x |= t.data_ptr()
    return 4096 if x == 0 else min(x & -x, 4096)


def workspace_bytes(m: int, n: int, k: int, cfg: int = CFG_AUTO, scaled: bool = False, ptr_align: int = 256) -> int:
    """Bytes of workspace the GEMM of this shape can use (0: it would not split K)."""
    return int(library().qm_gemm_workspace_bytes(m, n, k, ptr_align, cfg, 1 if scaled else 0))


def _workspace(workspace, a, b, m, n, k, cfg, scaled):
    """(pointer, bytes, keep-alive) of the workspace argument: True = allocate what the call
    can use from torch's caching allocator (stream-ordered, so safe across streams and under
    graph capture), None / False = none, a tensor = the caller's own."""
    if workspace is None or workspace is False:
        return None, 0, None
    if workspace is True:
        need = workspace_bytes(m, n, k, cfg, scaled, _ptr_align(a, b))
        if need == 0:
            return None, 0, None
        workspace = torch.empty((need,), dtype=torch.uint8, device=a.device)
    if not (isinstance(workspace, torch.Tensor) and workspace.is_cuda and workspace.device == a.device and workspace.is_contiguous()):
        raise QuadmulError("gemm: workspace must be a contiguous tensor on a's device")
    return workspace.data_ptr(), workspace.numel() * workspace.element_size(), workspace


def gemm_cfg(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor, m: int, n: int, k: int, cfg: int = CFG_AUTO,
             workspace=True) -> None:
    """``c[m,n] = a[m,k] @ b[n,k].T`` on packed int4, with an explicit kernel configuration.

    ``cfg``: config id in the low 16 bits, tile-raster group height in bits 16..23
    (0 = default), K split in bits 24..29; ``CFG_AUTO`` = table / cost model.
    ``workspace``: see :func:`gemm`.
    """
    _check_operands(a, b, c, m, n, k)
    ws, ws_bytes, _keep = _workspace(workspace, a, b, m, n, k, cfg, False)
    with torch.cuda.device(a.device):
        st = library().qm_gemm_i4_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, n, k, _stream_ptr(a), cfg, ws, ws_bytes)
    _check(st, "qm_gemm_i4_ws")


def gemm_scaled(a: torch.Tensor, b: torch.Tensor, d: torch.Tensor, m: int, n: int, k: int,
                row_scale: Optional[torch.Tensor] = None, col_scale: Optional[torch.Tensor] = None, cfg: int = CFG_AUTO,
                workspace=True) -> None:
    """The GEMM with the dequantising epilogue fused in (no counterpart in the reference's
    code; README.md:7 names the idea): ``d[m,n] = round(((float)c[m,n] * row_scale[m]) *
    col_scale[n])`` with ``c`` the exact int32 product; ``d`` is float16 or bfloat16 and is
    overwritten; the scales are float32 vectors on the same device, None = all ones.
    ``workspace``: see :func:`gemm`."""
    _check_operands(a, b, d, m, n, k, c_dtypes=(torch.float16, torch.bfloat16))
    for s_, cnt, what in ((row_scale, m, "row_scale"), (col_scale, n, "col_scale")):
        if s_ is None:
            continue
        if not (s_.is_cuda and s_.device == a.device and s_.dtype == torch.float32 and s_.is_contiguous() and s_.numel() == cnt):
            raise QuadmulError(f"gemm_scaled: {what} must be a contiguous float32 vector of {cnt} elements on a's device")
    out = 1 if d.dtype == torch.float16 else 2
    ws, ws_bytes, _keep = _workspace(workspace, a, b, m, n, k, cfg, True)
    with torch.cuda.device(a.device):
        st = library().qm_gemm_i4_scaled_ws(a.data_ptr(), b.data_ptr(), d.data_ptr(), m, n, k,
                                            None if row_scale is None else row_scale.data_ptr(),
                                            None if col_scale is None else col_scale.data_ptr(), out, _stream_ptr(a), cfg,
                                            ws, ws_bytes)
    _check(st, "qm_gemm_i4_scaled_ws")


def quantize_pack(x: torch.Tensor):
    """Per-row symmetric int4 quantisation fused with the packing, on the GPU (no counterpart
    in the reference; the packing half is pack_b, test.py:6-15).  ``x``: [rows, k] float16,
    bfloat16 or float32, contiguous.  Returns ``(packed int8 [rows, k/2], scales float32
    [rows])`` with ``scales = amax / 7`` -- the ``row_scale`` of ``gemm_scaled``."""
    if not (x.is_cuda and x.dim() == 2 and x.is_contiguous()):
        raise QuadmulError("quantize_pack: x must be a contiguous 2-d GPU tensor")
    kinds = {torch.float16: 1, torch.bfloat16: 2, torch.float32: 3}
    if x.dtype not in kinds:
        raise QuadmulError("quantize_pack: x must be float16, bfloat16 or float32")
    rows, k = x.shape
    if k % 2:
        raise QuadmulError("quantize_pack: k must be even")
    packed = torch.empty((rows, k // 2), dtype=torch.int8, device=x.device)
    scales = torch.empty((rows,), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        st = library().qm_quantize_pack_i4(x.data_ptr(), kinds[x.dtype], packed.data_ptr(), scales.data_ptr(), rows, k, _stream_ptr(x))
    _check(st, "qm_quantize_pack_i4")
    return packed, scales


def config_has_scaled(cfg: int) -> bool:
    """Whether configuration ``cfg`` exists with the scaled 16-bit float output."""
    return bool(library().qm_config_has_scaled(cfg))


def gemm(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor, m: int, n: int, k: int, workspace=True) -> None:
    """Same contract as the reference's ``quadmul.gemm`` (extension.cpp:8-24): ``a`` is
    packed A ``[m, k/2]``, ``b`` is packed B stored ``[n, k/2]``, ``c`` is ``[m, n]`` int32
    and is overwritten; enqueued on the current stream of ``a``'s device; returns None.

    ``workspace``: True (default) takes a temporary buffer from torch's allocator when the
    shape runs with K split over several workgroups per tile (few tiles, long K); None runs
    without one (the splits then meet in ``c`` through atomics); a uint8 tensor is used as
    it is.  The result is the same in every case."""
    gemm_cfg(a, b, c, m, n, k, CFG_AUTO, workspace)


STATIC_SCRATCH_BYTES = 64 << 20


def gemm_static(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor, m: int, n: int, k: int) -> None:
    """:func:`gemm` through ``qm_gemm_i4_static``: nothing is allocated, the scratch memory of
    a K split or of zero-padded operand copies is an array inside the library (at most
    ``STATIC_SCRATCH_BYTES``; beyond that the call raises).  Calls that may overlap on one GPU
    race on that array: keep them on one stream."""
    _check_operands(a, b, c, m, n, k)
    with torch.cuda.device(a.device):
        st = library().qm_gemm_i4_static(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, n, k, _stream_ptr(a))
    _check(st, "qm_gemm_i4_static")


def pack_int4(values: torch.Tensor) -> torch.Tensor:
    """``[rows, K]`` int8 holding int4 values -> ``[rows, K/2]`` int8, even k in the low
    nibble: the reference's ``pack_b`` (test.py:6-15).  GPU tensors are packed by the
    library's kernel, CPU tensors with the same bit arithmetic in torch."""
    if values.dtype != torch.int8 or values.dim() != 2:
        raise QuadmulError("pack_int4: expects a 2-D int8 tensor")
    rows, k = values.shape
    if k % 2:
        raise QuadmulError("pack_int4: K must be even")
    v = values.contiguous()
    if v.is_cuda:
        out = torch.empty((rows, k // 2), dtype=torch.int8, device=v.device)
        with torch.cuda.device(v.device):
            st = library().qm_pack_i4(v.data_ptr(), out.data_ptr(), rows, k, _stream_ptr(v))
        _check(st, "qm_pack_i4")
        return out
    u = v.view(torch.uint8).reshape(-1)
    return ((u[0::2] & 0x0F) | ((u[1::2] & 0x0F) << 4)).reshape(rows, k // 2).view(torch.int8).contiguous()


def unpack_int4(packed: torch.Tensor) -> torch.Tensor:
    """``[rows, K/2]`` bytes -> ``[rows, K]`` int8: the reference's ``unpack_int4_matrix``
    (kernel.cu:389-408)."""
    if not _is_byte(packed) or packed.dim() != 2:
        raise QuadmulError("unpack_int4: expects a 2-D int8/uint8 tensor")
    p = packed.contiguous()
    rows, half = p.shape
    if p.is_cuda:
        out = torch.empty((rows, 2 * half), dtype=torch.int8, device=p.device)
        with torch.cuda.device(p.device):
            st = library().qm_unpack_i4(p.data_ptr(), out.data_ptr(), rows, 2 * half, _stream_ptr(p))
        _check(st, "qm_unpack_i4")
        return out
    u = p.view(torch.uint8)
    lo = (u & 0x0F).to(torch.int16)
    hi = (u >> 4).to(torch.int16)
    lo = torch.where(lo > 7, lo - 16, lo)
    hi = torch.where(hi > 7, hi - 16, hi)
    return torch.stack((lo, hi), dim=2).reshape(rows, 2 * half).to(torch.int8)


def init(device=None) -> None:
    """Every kernel's one-off set-up on ``device`` (default: the current one) without launching
    anything; optional -- first launches do it by themselves."""
    with torch.cuda.device(device if device is not None else torch.cuda.current_device()):
        _check(library().qm_init(), "qm_init")


def num_configs() -> int:
    return int(library().qm_num_configs())


def config_name(cfg: int) -> str:
    s = library().qm_config_name(cfg)
    if s is None:
        raise QuadmulError(f"no kernel configuration {cfg}")
    return s.decode()


def config_names() -> List[str]:
    return [config_name(i) for i in range(num_configs())]


def config_id(name: str) -> int:
    names = config_names()
    if name not in names:
        raise QuadmulError(f"no kernel configuration named {name!r}")
    return names.index(name)


def select_config(m: int, n: int, k: int, ptr_align: int = 256) -> int:
    """The (config id | group_m << 16) ``gemm`` would use for this shape."""
    v = int(library().qm_select_config(m, n, k, ptr_align))
    if v < 0:
        _check(v, "qm_select_config")
    return v


def select_config_ex(m: int, n: int, k: int, ptr_align: int = 256, workspace: bool = True, scaled: bool = False) -> int:
    """The choice for any form of the call: with or without a workspace, int32 or scaled output."""
    v = int(library().qm_select_config_ex(m, n, k, ptr_align, 1 if workspace else 0, 1 if scaled else 0))
    if v < 0:
        _check(v, "qm_select_config_ex")
    return v


def config_supports(cfg: int, m: int, n: int, k: int, ptr_align: int = 256) -> bool:
    return bool(library().qm_config_supports(cfg, m, n, k, ptr_align))


def debug_set_operand_limit(nbytes: int) -> int:
    """Testing aid: operands of ``nbytes`` or more are cut into blocks (0 restores 2 GiB - 1);
    returns the previous limit.  See ``qm_debug_set_operand_limit`` in include/qm_abi.h."""
    return int(library().qm_debug_set_operand_limit(nbytes))


def version() -> str:
    return library().qm_version().decode()
