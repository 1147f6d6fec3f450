"""SwiGLU feed-forward: x += (silu(h Wg^T) * (h Wu^T)) Wd^T, gate and up rows stacked so one
product computes both (crates/glassbox-core/src/model.rs:64-66,335-344)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import (FeedForward, PreNormed, TensorSpec, emit_target, needs_multiple_of_8, product, product_in_slices,
                   split_workspace)


class SwiGLU(FeedForward):
    replayable = True
    taped = True

    def __init__(self, width: int, intermediate: int, any_size: bool = False):
        """``any_size``: sizes that the bfloat16 matrix-core products do not take (no multiples of 8) are not refused but
        go through the plain product, unfused."""
        self.width, self.intermediate, self.any_size = width, intermediate, bool(any_size)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"gate_proj.weight": TensorSpec((self.intermediate, self.width)),
                "up_proj.weight": TensorSpec((self.intermediate, self.width)),
                "down_proj.weight": TensorSpec((self.width, self.intermediate))}

    def load(self, tensors):
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], 0)
        self.w_down = tensors["down_proj.weight"].contiguous()

    def streamed_matrices(self):
        return [self.w_gate_up, self.w_down]

    def problems(self, dtype, page_size):
        if self.any_size:
            return []
        return needs_multiple_of_8(dtype, "width", self.width) + needs_multiple_of_8(dtype, "intermediate", self.intermediate)

    accepts_fused_norm = True
    accepts_emit_norm = True
    accepts_store = True

    def forward(self, ctx, h, residual, norm=None, emit=None, store: bool = False):
        """``norm=(gamma, eps)``: h is the un-normed float32 residual and the first product norms it;
        ``norm=PreNormed``: the product before has done most of that.  ``emit=(gamma, eps)``: the down
        projection may prepare the norm that reads the residual next (returns a PreNormed or Normed if it did).
        ``store``: the rows are written to ``residual`` (float32) instead of added."""
        n = h.shape[0]
        act = ctx.buffer("act", (n, self.intermediate), ctx.dtype)
        if ctx.dtype == torch.bfloat16 and (self.width % 8 or self.intermediate % 8):
            # (only with ``any_size``, and then without norms to fuse: the blocks that offer those build it without)
            gate_up = ctx.buffer("gate_up", (n, 2 * self.intermediate), ctx.dtype)
            product(ctx, h, self.w_gate_up, gate_up)
            ops.silu_mul(gate_up, act)
            product(ctx, act, self.w_down, residual, accumulate=not store)
            return None
        if isinstance(norm, PreNormed):
            ops.gemm(norm.rows, self.w_gate_up, act, silu_mul=True, rms_parts=norm.as_gemm_arg())
        elif ctx.dtype == torch.bfloat16 and self.intermediate % 8 == 0:
            # the activation is applied where the product's tile is finished: gate_up never reaches memory
            ops.gemm(h, self.w_gate_up, act, silu_mul=True, rms=norm,
                     workspace=None if norm is not None else split_workspace(ctx, n, 2 * self.intermediate, self.width))
        else:
            if norm is not None:   # nothing to fuse it into here: the norm gets its own pass after all
                normed = ctx.buffer("h", (n, self.width), ctx.dtype)
                ops.rmsnorm(h, norm[0], norm[1], normed)
                h = normed
            gate_up = ctx.buffer("gate_up", (n, 2 * self.intermediate), ctx.dtype)
            ops.gemm(h, self.w_gate_up, gate_up)
            ops.silu_mul(gate_up, act)
        target, handed_on = emit_target(ctx, n, self.width, self.intermediate, None if store else emit, "ffn")
        ops.gemm(act, self.w_down, residual, accumulate=not store, emit=target,
                 workspace=split_workspace(ctx, n, self.width, self.intermediate))
        return handed_on


class ClampedGLU(FeedForward):
    """A gated unit whose halves are clamped: g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit),
    y = g * sigmoid(alpha * g) * (u + 1), output W_down y.  Gate and up rows are stacked so one product computes both;
    its sums stay 32-bit until the unit has been applied."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, intermediate: int, limit: float, alpha: float = 1.702):
        self.width, self.intermediate = width, intermediate
        self.limit, self.alpha = float(limit), float(alpha)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"gate": TensorSpec((self.intermediate, self.width)), "up": TensorSpec((self.intermediate, self.width)),
                "down": TensorSpec((self.width, self.intermediate))}

    def load(self, tensors):
        self.w_gate_up = torch.cat([tensors["gate"], tensors["up"]], 0)
        self.w_down = tensors["down"].contiguous()

    def streamed_matrices(self):
        return [self.w_gate_up, self.w_down]

    def forward(self, ctx, h, residual, store: bool = False):
        n = h.shape[0]
        act = ctx.buffer("act", (n, self.intermediate), ctx.dtype)
        if ctx.dtype == torch.bfloat16 and ops.gemm_takes(h, self.w_gate_up):
            # the unit is applied where the product's tile is finished: gate_up never reaches memory
            ops.gemm_glu(h, self.w_gate_up, act, self.limit, self.alpha)
        else:
            gate_up = ctx.buffer("glu_gate_up", (n, 2 * self.intermediate), torch.float32)
            product(ctx, h, self.w_gate_up, gate_up)
            ops.glu_clamped(gate_up, act, self.limit, self.alpha)
        if store:   # the caller's norm adds the slices of a product that divides k
            return product_in_slices(ctx, act, self.w_down, residual)
        product(ctx, act, self.w_down, residual, accumulate=True)
        return None


class PolyNormMLP(FeedForward):
    """W_down act(W_up h) without a gate; act is a polynomial of normed powers, a N(z) + b N(z^2) + c N(z^3) + e with
    the powers taken element by element and N(v) = v / sqrt(mean(v^2) + eps) over a token's ``intermediate`` values;
    ``act`` holds a, b, c, e.  The sums are 32-bit."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, intermediate: int, eps: float):
        self.width, self.intermediate, self.eps = width, intermediate, float(eps)
        self.w_up = self.w_down = self.coef = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"up": TensorSpec((self.intermediate, self.width)), "down": TensorSpec((self.width, self.intermediate)),
                "act": TensorSpec((4,), kind="f32", init="ones")}

    def load(self, tensors):
        self.w_up, self.w_down = tensors["up"].contiguous(), tensors["down"].contiguous()
        self.coef = tensors["act"].float().contiguous()

    def streamed_matrices(self):
        return [self.w_up, self.w_down]

    def forward(self, ctx, h, residual, store: bool = False):
        n = h.shape[0]
        z = ctx.buffer("poly_z", (n, self.intermediate), ctx.dtype)
        product(ctx, h, self.w_up, z)
        act = ctx.buffer("act", (n, self.intermediate), ctx.dtype)
        ops.poly_norm(z, self.coef, self.eps, act)
        if store:   # the caller's norm adds the slices of a product that divides k
            return product_in_slices(ctx, act, self.w_down, residual)
        product(ctx, act, self.w_down, residual, accumulate=True)
        return None
