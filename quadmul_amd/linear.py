"""A W4A4 linear layer on top of the packed-int4 GEMM: the caller the reference's README
(README.md:7, "easy to fuse with quantisation") has in mind and does not ship.

    y[t, n] = round16((sum_k xq[t, k] * wq[n, k]) * x_scale[t] * w_scale[n]) (+ bias[n])

with ``xq, x_scale = quantize_pack(x)`` (per-token symmetric int4, scale = amax / 7) and
``wq, w_scale`` the same quantisation of the weight rows, done once.  Three launches per
call: quantise + pack the activations, the GEMM with the dequantising epilogue, and the
bias add when there is one; the int32 product never reaches memory.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import QuadmulError, gemm_scaled, quantize_pack


class W4A4Linear(torch.nn.Module):
    """``forward(x)``: ``x`` [..., in_features] float16 / bfloat16 / float32 on the GPU ->
    [..., out_features] in ``out_dtype`` (float16 or bfloat16)."""

    def __init__(self, weight_packed: torch.Tensor, weight_scale: torch.Tensor, bias: Optional[torch.Tensor] = None,
                 out_dtype: torch.dtype = torch.float16):
        super().__init__()
        if weight_packed.dim() != 2 or weight_packed.dtype not in (torch.int8, torch.uint8):
            raise QuadmulError("W4A4Linear: weight_packed must be [out_features, in_features / 2] int8 or uint8")
        if out_dtype not in (torch.float16, torch.bfloat16):
            raise QuadmulError("W4A4Linear: out_dtype must be float16 or bfloat16")
        n = weight_packed.shape[0]
        if weight_scale.shape != (n,) or weight_scale.dtype != torch.float32:
            raise QuadmulError("W4A4Linear: weight_scale must be float32 [out_features]")
        if bias is not None and bias.shape != (n,):
            raise QuadmulError("W4A4Linear: bias must be [out_features]")
        self.out_features = n
        self.in_features = weight_packed.shape[1] * 2
        self.out_dtype = out_dtype
        self.register_buffer("weight_packed", weight_packed.contiguous())
        self.register_buffer("weight_scale", weight_scale.contiguous())
        self.register_buffer("bias", None if bias is None else bias.to(out_dtype).contiguous())

    @classmethod
    def from_float(cls, weight: torch.Tensor, bias: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.float16):
        """Quantise a float [out_features, in_features] weight (on the GPU) row by row with the
        library's own kernel: the same rule as for the activations."""
        wq, ws = quantize_pack(weight.contiguous())
        return cls(wq, ws, bias, out_dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.shape[-1] != self.in_features:
            raise QuadmulError(f"W4A4Linear: last dimension of x must be {self.in_features}")
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.in_features)
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        m = x2.shape[0]
        y = torch.empty((m, self.out_features), dtype=self.out_dtype, device=x.device)
        if m:
            xq, xs = quantize_pack(x2)
            gemm_scaled(xq, self.weight_packed, y, m, self.out_features, self.in_features, xs, self.weight_scale)
            if self.bias is not None:
                y += self.bias
        return y.reshape(*lead, self.out_features)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, out_dtype={self.out_dtype}"
