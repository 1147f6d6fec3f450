"""Arrangement of a layer's parts.  PreNormBlock is the Llama arrangement: norm, mixer, add;
norm, feed-forward, add (crates/glassbox-core/src/model.rs:251-344).  The residual stream is
float32 in both precisions; mixer and feed-forward add into it themselves.

A mixer or feed-forward with ``accepts_fused_norm = True`` may be handed the un-normed residual
and the norm's constants instead of normed rows (``forward(..., norm=(gamma, eps))``): its first
matrix product then computes the norm on the way (few rows only; ``Norm.fuse_spec`` decides).
With ``accepts_emit_norm = True`` it may also be asked to prepare the norm that reads the residual
after it (``forward(..., emit=(gamma, eps))``, returning a ``PreNormed``, or a ``Normed`` if its product
did the whole norm): then the norm's pass over the residual happens where the residual is made, inside a
block and from one block to the next (``Norm.emit_spec`` says whether the norm allows it)."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import Block, CacheSpec, FeedForward, LayerCache, Mixer, Norm, Normed, Part, StateSpec


class PreNormBlock(Block):
    replayable = True
    taped = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, ffn_norm: Norm, ffn: FeedForward,
                 names=("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.names = tuple(names)

    def children(self) -> Dict[str, Part]:
        return dict(zip(self.names, (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)))

    def cache_spec(self) -> Optional[CacheSpec]:
        return self.mixer.cache_spec

    def state_spec(self) -> Optional[StateSpec]:
        return self.mixer.state_spec

    def entry_norm(self, ctx, n: int):
        """``(gamma, eps)`` of the norm this block begins with, if the product that made the residual before
        it may prepare that norm or do it (``forward(..., pre=)`` then takes what it made); else None."""
        return self.mixer_norm.emit_spec(ctx, n) if getattr(self.mixer, "accepts_fused_norm", False) else None

    def forward(self, ctx, x, cache: Optional[LayerCache], pre=None, emit=None):
        """``pre``: a PreNormed or Normed for this block's first norm, from the block before; ``emit``: the
        ``entry_norm`` of the block after.  Returns a PreNormed or Normed for that block if the feed-forward made one."""
        n = x.shape[0]
        fused = getattr(self.mixer, "accepts_fused_norm", False)
        ffn_fused = getattr(self.ffn, "accepts_fused_norm", False)
        more = {}
        if ffn_fused and getattr(self.mixer, "accepts_emit_norm", False):
            more["emit"] = self.ffn_norm.emit_spec(ctx, n)
        if isinstance(pre, Normed):   # the norm is done: its rows come in its place
            mid = self.mixer.forward(ctx, pre.rows, x, cache, **more)
        else:
            spec = (pre if pre is not None else self.mixer_norm.fuse_spec(ctx, n)) if fused else None
            if spec is not None:
                mid = self.mixer.forward(ctx, x, x, cache, norm=spec, **more)
            else:
                mid = self.mixer.forward(ctx, self.mixer_norm.forward(ctx, x), x, cache, **more)
        more = {"emit": emit} if emit is not None and getattr(self.ffn, "accepts_emit_norm", False) else {}
        if isinstance(mid, Normed):
            return self.ffn.forward(ctx, mid.rows, x, **more)
        spec = (mid if mid is not None else self.ffn_norm.fuse_spec(ctx, n)) if ffn_fused else None
        if spec is not None:
            return self.ffn.forward(ctx, x, x, norm=spec, **more)
        return self.ffn.forward(ctx, self.ffn_norm.forward(ctx, x), x, **more)


class MixerOnlyBlock(Block):
    """A layer without a feed-forward: norm, mixer, add."""
    replayable = True
    taped = True

    def __init__(self, mixer_norm: Norm, mixer: Mixer, names=("norm1", "mix")):
        self.mixer_norm, self.mixer = mixer_norm, mixer
        self.names = tuple(names)

    def children(self) -> Dict[str, Part]:
        return dict(zip(self.names, (self.mixer_norm, self.mixer)))

    def cache_spec(self) -> Optional[CacheSpec]:
        return self.mixer.cache_spec

    def state_spec(self) -> Optional[StateSpec]:
        return self.mixer.state_spec

    def forward(self, ctx, x, cache: Optional[LayerCache]):
        self.mixer.forward(ctx, self.mixer_norm.forward(ctx, x), x, cache)
        return None


class ParallelBlock(Block):
    """One norm, and both sublayers read its rows: x += mult * (mixer(norm(x)) + feed-forward(norm(x))); the
    feed-forward may be absent.  The sublayers' sum is made in a 32-bit buffer of its own (the mixer writes its rows
    there, the feed-forward adds to them: ``accepts_store``) and goes into the residual in one pass."""
    replayable = True
    taped = True

    def __init__(self, norm: Norm, mixer: Mixer, ffn: Optional[FeedForward] = None, mult: float = 1.0,
                 names=("norm1", "mix", "mlp")):
        for part in (mixer,):
            if not getattr(part, "accepts_store", False):
                raise ValueError(f"{type(part).__name__} cannot write its rows instead of adding them (accepts_store)")
        self.norm, self.mixer, self.ffn = norm, mixer, ffn
        self.mult = float(mult)
        self.names = tuple(names)

    def children(self) -> Dict[str, Part]:
        out = {self.names[0]: self.norm, self.names[1]: self.mixer}
        if self.ffn is not None:
            out[self.names[2]] = self.ffn
        return out

    def cache_spec(self) -> Optional[CacheSpec]:
        return self.mixer.cache_spec

    def state_spec(self) -> Optional[StateSpec]:
        return self.mixer.state_spec

    def forward(self, ctx, x, cache: Optional[LayerCache]):
        n, width = x.shape
        h = self.norm.forward(ctx, x)
        y = ctx.buffer("parallel_y", (n, width), torch.float32)
        self.mixer.forward(ctx, h, y, cache, store=True)
        if self.ffn is not None:
            self.ffn.forward(ctx, h, y)
        ops.axpy_rows(x, y, self.mult)
        return None


class OutputNormBlock(Block):
    """A layer that norms what its sublayers give back, not what they read: x += norm1(mixer(conv(x))), then
    x += norm2(feed-forward(x)); the
    feed-forward may be absent.  The sublayers read the residual itself (the mixer through ``conv``, which may add a short
    convolution of the residual over time and keeps the state that takes); each writes its rows into a 32-bit buffer
    (``accepts_store``), and the norm's pass over them is the pass that adds them into the residual.  The norms are
    ``ScalarRMSNorm``s (or anything with ``add_normed``)."""
    replayable = True
    taped = True

    def __init__(self, conv, mixer: Mixer, mixer_norm, ffn: Optional[FeedForward] = None, ffn_norm=None,
                 names=("canon1", "mix", "norm1", "mlp", "norm2")):
        for part in (mixer, ffn):
            if part is not None and not getattr(part, "accepts_store", False):
                raise ValueError(f"{type(part).__name__} cannot write its rows instead of adding them (accepts_store)")
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        if conv.state_spec is not None and mixer.state_spec is not None:
            raise ValueError("the convolution and the mixer both keep state: a cache layer has one state")
        self.conv, self.mixer, self.mixer_norm, self.ffn, self.ffn_norm = conv, mixer, mixer_norm, ffn, ffn_norm
        self.names = tuple(names)

    def children(self) -> Dict[str, Part]:
        out = {self.names[0]: self.conv, self.names[1]: self.mixer, self.names[2]: self.mixer_norm}
        if self.ffn is not None:
            out[self.names[3]] = self.ffn
            out[self.names[4]] = self.ffn_norm
        return out

    def cache_spec(self) -> Optional[CacheSpec]:
        return self.mixer.cache_spec

    def state_spec(self) -> Optional[StateSpec]:
        return self.conv.state_spec if self.conv.state_spec is not None else self.mixer.state_spec

    def entry_rows(self, ctx, n: int, cache: Optional[LayerCache]):
        """``(weight, state)`` of the convolution this block begins with, if the pass that makes the residual before
        it may also make the rows this block's mixer reads (``forward(..., pre=)`` then takes them): a step of
        single tokens, whose rows need nothing of the step's other rows; else None."""
        return self.conv.entry_spec(ctx, n, cache) if hasattr(self.conv, "entry_spec") else None

    def forward(self, ctx, x, cache: Optional[LayerCache], pre=None, emit=None):
        """``pre``: the rows this block's mixer reads, made by the block before; ``emit``: the ``entry_rows`` of the block
        after.  Returns the rows for that block if the last norm's pass made them."""
        n, width = x.shape
        h = pre if pre is not None else self.conv.forward(ctx, x, cache)
        y = ctx.buffer("sublayer_y", (n, width), torch.float32)
        # a sublayer's rows lie in y, or in slices that the norm's pass adds up (``product_in_slices``)
        made, slices = self.mixer.forward(ctx, h, y, cache, store=True) or (y, 1)
        handed = ctx.buffer("h", (n, width), ctx.dtype) if emit is not None else None
        if self.ffn is None:
            self.mixer_norm.add_normed(ctx, made, x, rounded=handed, slices=slices, conv=emit)
            return handed
        if ctx.dtype == torch.float32:
            self.mixer_norm.add_normed(ctx, made, x, slices=slices)
            rows = x
        else:   # the pass that makes the residual also leaves it in the activations' type for the feed-forward
            rows = ctx.buffer("h", (n, width), ctx.dtype)
            self.mixer_norm.add_normed(ctx, made, x, rounded=rows, slices=slices)
        made, slices = self.ffn.forward(ctx, rows, y, store=True) or (y, 1)
        self.ffn_norm.add_normed(ctx, made, x, rounded=handed, slices=slices, conv=emit)
        return handed


class SandwichBlock(Block):
    """Every sublayer between two norms: x += norm1b(mixer(norm1(x))), then x += norm2b(feed-forward(norm2(x))); the
    feed-forward (with its two norms) may be absent.  The sublayers write their rows into a 32-bit buffer
    (``accepts_store``) or leave them in the slices of a product that divides k, and the pass of the norm behind a
    sublayer is the pass that adds into the residual.  The norms are ``TanhNorm``s (or anything with ``add_normed(ctx, y,
    x, slices=, then=, rounded=)``): a norm that needs no statistic of the row can also be applied to the new residual in
    that same pass, so the rows the feed-forward reads, and the rows the next block's mixer reads, come out of the pass
    before them."""
    replayable = True
    taped = True

    def __init__(self, norm1, mixer: Mixer, norm1b, norm2=None, ffn: Optional[FeedForward] = None, norm2b=None,
                 names=("norm1", "mix", "norm1b", "norm2", "mlp", "norm2b")):
        for part in (mixer, ffn):
            if part is not None and not getattr(part, "accepts_store", False):
                raise ValueError(f"{type(part).__name__} cannot write its rows instead of adding them (accepts_store)")
        if not ((ffn is None) == (norm2 is None) == (norm2b is None)):
            raise ValueError("a feed-forward and its two norms come together")
        self.norm1, self.mixer, self.norm1b, self.norm2, self.ffn, self.norm2b = norm1, mixer, norm1b, norm2, ffn, norm2b
        self.names = tuple(names)

    def children(self) -> Dict[str, Part]:
        parts = (self.norm1, self.mixer, self.norm1b, self.norm2, self.ffn, self.norm2b)
        return {name: part for name, part in zip(self.names, parts) if part is not None}

    def cache_spec(self) -> Optional[CacheSpec]:
        return self.mixer.cache_spec

    def state_spec(self) -> Optional[StateSpec]:
        return self.mixer.state_spec

    def entry_rows(self, ctx, n: int, cache: Optional[LayerCache]):
        """``(alpha, weight, bias)`` of the norm this block begins with, if the pass that makes the residual before it may
        also make the rows this block's mixer reads (``forward(..., pre=)`` then takes them); else None."""
        return self.norm1.spec() if hasattr(self.norm1, "spec") else None

    def forward(self, ctx, x, cache: Optional[LayerCache], pre=None, emit=None):
        """``pre``: the rows this block's mixer reads, made by the block before; ``emit``: the ``entry_rows`` of the block
        after.  Returns the rows for that block if the last norm's pass made them."""
        n, width = x.shape
        h = pre if pre is not None else self.norm1.forward(ctx, x)
        y = ctx.buffer("sublayer_y", (n, width), torch.float32)
        made, slices = self.mixer.forward(ctx, h, y, cache, store=True) or (y, 1)
        handed = ctx.buffer("h_handed", (n, width), ctx.dtype) if emit is not None else None
        if self.ffn is None:
            self.norm1b.add_normed(ctx, made, x, slices=slices, then=emit, rounded=handed)
            return handed
        rows = ctx.buffer("h", (n, width), ctx.dtype)
        self.norm1b.add_normed(ctx, made, x, slices=slices, then=self.norm2.spec(), rounded=rows)
        made, slices = self.ffn.forward(ctx, rows, y, store=True) or (y, 1)
        self.norm2b.add_normed(ctx, made, x, slices=slices, then=emit, rounded=handed)
        return handed
