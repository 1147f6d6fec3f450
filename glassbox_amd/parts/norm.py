"""RMS norm: out = g * (x / sqrt(mean(x^2) + eps)), sums in 32-bit
(crates/glassbox-core/src/model.rs:94-100).  With ``offset`` the checkpoint holds the weight minus ``offset`` and
g = offset + w, added in 32-bit when the weights are loaded and kept in 32-bit.  ``ScalarRMSNorm`` has one number for all
coordinates and can also norm a sublayer's *output* on its way into the residual.  ``TanhNorm`` computes no statistic
of the row at all: out = tanh(alpha x) * w + b with one number alpha."""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .. import ops
from .base import Norm, TensorSpec


class RMSNorm(Norm):
    replayable = True
    taped = True

    def __init__(self, width: int, eps: float, offset: float = 0.0):
        self.width = width
        self.eps = float(eps)
        self.offset = float(offset)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        if self.offset:
            # (offset + w rounded to bfloat16 would lose most of w: the sum stays 32-bit)
            return {"weight": TensorSpec((self.width,), kind="f32", init="zeros")}
        return {"weight": TensorSpec((self.width,), kind="vector", init="ones")}

    def load(self, tensors):
        w = tensors["weight"]
        self.weight = (w.float() + self.offset).contiguous() if self.offset else w.contiguous()

    def forward(self, ctx, x, rows=None, out_name="h"):
        m = x.shape[0] if rows is None else rows.numel()
        out = ctx.buffer(out_name, (m, self.width), ctx.dtype)
        ops.rmsnorm(x, self.weight, self.eps, out, rows)
        return out

    def emit_spec(self, ctx, n: int) -> Optional[Tuple[torch.Tensor, float]]:
        """(gamma, eps) if the product that makes the residual may prepare or do this norm (bfloat16 steps)."""
        if ctx.dtype == torch.bfloat16 and ctx.fuse_norms:
            return (self.weight, self.eps)
        return None

    def fuse_spec(self, ctx, n: int) -> Optional[Tuple[torch.Tensor, float]]:
        """(gamma, eps) if the next matrix product may compute this norm itself: bfloat16 steps of
        few rows, where a pass of its own costs more than the norm's arithmetic."""
        if ctx.dtype == torch.bfloat16 and n <= ops.FUSED_NORM_MAX_ROWS and ctx.fuse_norms:
            return (self.weight, self.eps)
        return None


class ScalarRMSNorm(Norm):
    """out = g * (x / sqrt(mean(x^2) + eps)) with a single number g (a tensor without dimensions).  As a norm of rows
    (``forward``: a final norm) it is the kernel of ``RMSNorm`` with g in every column; ``add_normed`` norms a
    sublayer's output y and adds it into the residual in one pass."""
    replayable = True
    taped = True

    def __init__(self, width: int, eps: float):
        self.width = width
        self.eps = float(eps)
        self.gain: Optional[torch.Tensor] = None      # [1]
        self.weight: Optional[torch.Tensor] = None    # [width], the same number

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((), kind="f32", init="ones")}

    def load(self, tensors):
        self.gain = tensors["weight"].float().reshape(1).contiguous()
        self.weight = self.gain.expand(self.width).contiguous()

    def forward(self, ctx, x, rows=None, out_name="h"):
        m = x.shape[0] if rows is None else rows.numel()
        out = ctx.buffer(out_name, (m, self.width), ctx.dtype)
        ops.rmsnorm(x, self.weight, self.eps, out, rows)
        return out

    def add_normed(self, ctx, y, x, rounded=None, slices: int = 1, conv=None) -> None:
        """x += g * y / sqrt(mean(y^2) + eps) (both float32; ``slices`` > 1: y is the sum of that many pieces);
        ``rounded`` receives the new x in its own type, or with ``conv=(weight, state)`` what a ``TimeConv`` makes of it."""
        ops.norm_add(x, y, self.gain, self.eps, rounded, slices=slices, conv=conv, ctx=ctx)


class TanhNorm(Norm):
    """out = tanh(alpha * x) * weight + bias: ``alpha`` a single number (a tensor without dimensions), weight and bias a
    number a coordinate; no mean, no variance.  As a norm of rows (``forward``) it writes the rows a sublayer reads;
    ``add_normed`` norms a sublayer's output y on its way into the residual, and since nothing of a row has to be
    summed first, the same pass can also write the rows that the next norm of this kind makes of the new residual
    (``then=``).  32-bit arithmetic in both precisions."""
    replayable = True
    taped = True

    def __init__(self, width: int):
        self.width = width
        self.alpha: Optional[torch.Tensor] = None     # [1]
        self.weight: Optional[torch.Tensor] = None    # [width]
        self.bias: Optional[torch.Tensor] = None      # [width]

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.width,), kind="f32", init="ones"),
                "bias": TensorSpec((self.width,), kind="f32", init="normal"),
                "alpha": TensorSpec((), kind="f32", init="ones")}

    def load(self, tensors):
        self.alpha = tensors["alpha"].float().reshape(1).contiguous()
        self.weight = tensors["weight"].float().contiguous()
        self.bias = tensors["bias"].float().contiguous()

    def spec(self) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        return (self.alpha, self.weight, self.bias)

    def forward(self, ctx, x, rows=None, out_name="h"):
        m = x.shape[0] if rows is None else rows.numel()
        out = ctx.buffer(out_name, (m, self.width), ctx.dtype)
        ops.tanh_norm(x, self.alpha, self.weight, self.bias, out, rows)
        return out

    def in_place(self, ctx, x) -> None:
        """x = norm(x) on float32 rows (an embedding's output)."""
        ops.tanh_norm(x, self.alpha, self.weight, self.bias, x)

    def add_normed(self, ctx, y, x, slices: int = 1, then: Optional[tuple] = None, rounded=None) -> None:
        """x += norm(y) (both float32; ``slices`` > 1: y is the sum of that many pieces); with ``then`` (the ``spec()`` of
        the norm that reads x next) and ``rounded``: rounded = that norm of the new x."""
        ops.tanh_norm_add(x, y, self.spec(), slices=slices, then=then, h=rounded)
