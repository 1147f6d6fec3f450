"""A short causal convolution over time on the residual itself: what a mixer reads is h = x + conv(x),
conv(x)[t] = sum_j w[:, j] x[t - taps + 1 + j] over the request's own tokens (``weight`` [width, taps], no bias, zeros
before the first token).  The request's last taps - 1 rows of x are its state, in 32-bit like the residual."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import LayerCache, Part, StateSpec, TensorSpec


class TimeConv(Part):
    replayable = True
    taped = True

    def __init__(self, width: int, taps: int):
        """``taps`` 0: no convolution, the rows are the residual rounded to the activations' type."""
        self.width, self.taps = int(width), int(taps)
        self.state_spec = StateSpec((self.taps - 1, self.width), torch.float32, 0.0) if self.taps > 1 else None
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.width, self.taps), kind="f32")} if self.taps else {}

    def load(self, tensors):
        if self.taps:
            self.weight = tensors["weight"].float().t().contiguous()   # a row a tap: neighbouring channels side by side

    def problems(self, dtype, page_size):
        if self.taps > ops.TIME_CONV_MAX_TAPS:
            return [("taps", f"{self.taps} is above {ops.TIME_CONV_MAX_TAPS}, the longest convolution the kernel takes")]
        return []

    def entry_spec(self, ctx, n: int, cache: Optional[LayerCache]):
        """``(weight, state)`` for ``ops.norm_add(conv=)`` if the pass that adds a normed sublayer into the residual may
        make this convolution's rows as well (every request of the step brings one row), else None."""
        if (not self.taps or int(ctx.host["max_q_len"]) != 1 or not ops.norm_add_takes_rows(self.width)
                or (self.taps > 1 and (cache is None or cache.state is None))):
            return None
        return (self.weight, cache.state if self.taps > 1 else None)

    def forward(self, ctx, x, cache: Optional[LayerCache], out_name: str = "h") -> torch.Tensor:
        """The rows a mixer reads, in the activations' type; moves the requests' state on (call it before x changes)."""
        if self.taps > 1 and (cache is None or cache.state is None):
            raise ValueError("TimeConv needs its state (the last rows of each request)")
        out = ctx.buffer(out_name, tuple(x.shape), ctx.dtype)
        ops.time_conv(x, self.weight, cache.state if self.taps > 1 else None, ctx, out)
        return out
