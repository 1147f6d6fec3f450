"""Token embedding (a row copy, crates/glassbox-core/src/model.rs:228-231) and the output head
(final norm on the wanted rows only, then the vocabulary product, model.rs:350-361; the head is
the embedding table when tied, model.rs:190-192)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import LayerCache, Part, StateSpec, TensorSpec, needs_multiple_of_8, product


class Embedding(Part):
    replayable = True

    def __init__(self, vocab: int, width: int, scale: float = 1.0, norm: Optional[Part] = None):
        self.vocab, self.width, self.scale = vocab, width, float(scale)
        #: a norm of the embedded rows, applied in place to the 32-bit rows (anything with ``in_place(ctx, x)``)
        self.norm = norm
        self.table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.vocab, self.width))}

    def children(self) -> Dict[str, Part]:
        return {"norm": self.norm} if self.norm is not None else {}

    def load(self, tensors):
        self.table = tensors["weight"].contiguous()

    def forward(self, ctx, out):
        """``out`` [n, width], or [streams, n, width]: every stream starts as the embedding."""
        ops.embed(self.table, ctx.token_ids, out, self.scale)
        if self.norm is not None:
            if out.dim() != 2:
                raise ValueError("a normed embedding fills one residual, not several streams")
            self.norm.in_place(ctx, out)


class PairHashEmbedding(Embedding):
    """The token's row plus a row of a second table chosen by the token and the one before it:
    row (previous token * mul_prev + token * mul_cur) mod buckets, and the table's last row (number ``buckets``) for a
    request's first token.  The token before a step's first row is part of the request's state: one int32 a slot
    (``state_spec``), which the model hands over as a cache layer of the embedding's own."""
    replayable = True

    def __init__(self, vocab: int, width: int, buckets: int, mul_prev: int, mul_cur: int,
                 names=("weight", "pairs")):
        super().__init__(vocab, width)
        if buckets < 1:
            raise ValueError(f"{buckets} buckets: at least one")
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        self.names = tuple(names)
        self.pairs: Optional[torch.Tensor] = None
        self.state_spec = StateSpec((1,), torch.int32, 0)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.names[0]: TensorSpec((self.vocab, self.width)),
                self.names[1]: TensorSpec((self.buckets + 1, self.width))}

    def load(self, tensors):
        self.table = tensors[self.names[0]].contiguous()
        self.pairs = tensors[self.names[1]].contiguous()

    def forward(self, ctx, out, cache: Optional[LayerCache] = None):
        if cache is None or cache.state is None:
            raise ValueError("PairHashEmbedding needs its state (the token before each request's step)")
        ops.embed_pairs(self.table, self.pairs, ctx, out, self.buckets, self.mul_prev, self.mul_cur, cache.state)


class LMHead(Part):
    """logits = rows . W^T (times ``scale``) in float32.  ``tied_to`` names an Embedding whose table is the head."""
    replayable = True

    def __init__(self, vocab: int, width: int, tied_to: Optional[Embedding] = None, scale: float = 1.0, any_size: bool = False):
        self.vocab, self.width, self.tied_to, self.scale = vocab, width, tied_to, float(scale)
        self.any_size = bool(any_size)   # a width that the bfloat16 product does not take goes through the plain product
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {} if self.tied_to is not None else {"weight": TensorSpec((self.vocab, self.width))}

    def load(self, tensors):
        if self.tied_to is None:
            self.weight = tensors["weight"].contiguous()

    def matrix(self) -> torch.Tensor:
        return self.tied_to.table if self.tied_to is not None else self.weight

    def streamed_matrices(self):
        return [self.matrix()]

    def problems(self, dtype, page_size):
        return [] if self.any_size else needs_multiple_of_8(dtype, "width", self.width)

    accepts_prepared = True

    def forward(self, ctx, rows, prepared=None):
        """``prepared``: a PreNormed whose rows these are: the product scales its result by the norm's factor."""
        logits = ctx.buffer("logits", (rows.shape[0], self.vocab), torch.float32)
        if prepared is None and not ops.gemm_takes(rows, self.matrix()):
            product(ctx, rows, self.matrix(), logits)
        else:
            ops.gemm(rows, self.matrix(), logits, rms_parts=prepared.as_gemm_arg() if prepared is not None else None)
        if self.scale != 1.0:
            ops.scale_rows(logits, self.scale)
        return logits
