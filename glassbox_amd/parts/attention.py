"""Grouped-query attention over the paged cache: the mixer of a Llama layer.

qkv = h . Wqkv^T (query rows, then key rows, then value rows stacked, as the
reference stacks them: crates/glassbox-core/src/model.rs:59-61,260-265);
positions are encoded and keys/values written to the pages
(model.rs:266-276); every token attends to its own request's positions up to
its own through the block table (model.rs:285-312); the output projection is
added into the residual (model.rs:322-325).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .. import ops
from .base import (FULL, RUNS, WINDOW, CacheSpec, LayerCache, Mixer, PositionEncoding, PreNormed, StateSpec, TensorSpec, emit_target,
                   needs_multiple_of_8, product, product_in_slices, split_workspace)


def paged_attention(ctx, q: torch.Tensor, out: torch.Tensor, cache: LayerCache, n_heads: int, scale: float,
                    window: int, keep_first: int = 0, chunk: int = 0, softcap: float = 0.0,
                    sinks: Optional[torch.Tensor] = None) -> None:
    """Attention of every row of the step over its request's pages.  ``window`` > 0: a token reads the last so many
    keys up to its own, and with ``keep_first`` the request's first so many keys as well, wherever they lie.
    ``chunk`` > 0 (instead of a window): positions are cut into runs of so many, counted from the request's first, and a
    token reads the keys of its own run up to itself.  ``softcap`` > 0: scores pass softcap * tanh(score / softcap).
    ``sinks`` (float32 [heads]): exp(sinks[h]) joins the softmax's denominator of head h and has no value.

    float32 always takes the plain kernel.  bfloat16 takes the tuned kernels where they apply: requests with
    one row go to the split-context decode kernel, longer portions to the matrix-core prefill kernel; a step
    with ``ctx.tuned`` off takes the plain kernel throughout."""
    if (ctx.dtype == torch.float32 or not ctx.tuned
            or not ops.tuned_attention_supports(cache.k_pages, n_heads, window, keep_first)):
        longest = int(ctx.host["max_context"])
        _, _, n_pieces, page_size, piece = cache.k_pages.shape
        tables = ctx.tables[cache.group]

        def rows(a, b, grouped):
            # few tokens with long contexts (a decode step): a workgroup a chunk of the context, merged by a second kernel
            floats = 0 if grouped else ops.attention_plain_split_floats(b - a, n_heads, n_pieces * piece, page_size, longest,
                                                                        keep_first)
            ws = ctx.buffer("attention_plain_parts", (floats,), torch.float32) if floats else None
            ops.attention_plain(q[a:b], out[a:b], ctx.positions[a:b], ctx.tok_seq[a:b], tables, cache.k_pages, cache.v_pages,
                                n_heads, scale, window, workspace=ws, max_context=longest, grouped=grouped,
                                keep_first=keep_first, chunk=chunk, softcap=softcap, sinks=sinks)

        # the rows of requests with one token come first; many rows of prompt portions go eight rows a workgroup
        n, n_decode = q.shape[0], ctx.host["n_decode"]
        if n - n_decode >= ops.PLAIN_GROUP_MIN_ROWS and window == 0 and chunk == 0:
            if n_decode > 0:
                rows(0, n_decode, False)
            rows(n_decode, n, True)
        else:
            rows(0, n, False)
        return
    n_decode = ctx.host["n_decode"]
    if n_decode > 0:
        ops.attention_decode(q, out, ctx, cache, n_heads, scale, window, keep_first, chunk, softcap, sinks)
    if n_decode < ctx.num_seqs:
        ops.attention_prefill(q, out, ctx, cache, n_heads, scale, window, keep_first, chunk, softcap, sinks)


class PagedAttention(Mixer):
    replayable = True
    taped = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, position: PositionEncoding,
                 window: int = 0, shares_kv: bool = False, scale: Optional[float] = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key heads")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.position = position
        self.window = int(window)
        self.shares_kv = shares_kv          # reads another layer's pages; has no key/value projections
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)  # model.rs:244
        self.q_dim = n_heads * head_dim
        self.kv_dim = n_kv_heads * head_dim
        self.cache_spec = None if shares_kv else CacheSpec(n_kv_heads, head_dim,
                                                           WINDOW if window > 0 else FULL, self.window)
        self.wqkv: Optional[torch.Tensor] = None
        self.wo: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {"q_proj.weight": TensorSpec((self.q_dim, self.width))}
        if not self.shares_kv:
            specs["k_proj.weight"] = TensorSpec((self.kv_dim, self.width))
            specs["v_proj.weight"] = TensorSpec((self.kv_dim, self.width))
        specs["o_proj.weight"] = TensorSpec((self.width, self.q_dim))
        return specs

    def children(self):
        return {"": self.position} if self.position.tensor_specs() else {}

    def all_replayable(self) -> bool:
        return self.replayable and self.position.all_replayable()

    def all_taped(self) -> bool:
        return self.taped and self.position.all_taped()

    def load(self, tensors):
        if self.shares_kv:
            self.wqkv = tensors["q_proj.weight"].contiguous()
        else:
            # one product computes all three (model.rs:59-61)
            self.wqkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], 0)
        self.wo = tensors["o_proj.weight"].contiguous()

    def streamed_matrices(self):
        return [self.wqkv, self.wo]

    def problems(self, dtype, page_size):
        out = needs_multiple_of_8(dtype, "width", self.width) + needs_multiple_of_8(dtype, "n_heads * head_dim", self.q_dim)
        if self.head_dim > ops.MAX_HEAD_DIM:
            out.append(("head_dim", f"{self.head_dim} is above {ops.MAX_HEAD_DIM}, the largest head the attention kernels take"))
        return out + self.position.problems(dtype, page_size)

    accepts_fused_norm = True
    accepts_emit_norm = True

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], norm=None, emit=None):
        """``norm=(gamma, eps)``: h is the un-normed float32 residual and the first product norms it;
        ``norm=PreNormed``: the product before has done most of that.  ``emit=(gamma, eps)``: the output
        projection may prepare the norm that reads the residual next (returns a PreNormed if it did)."""
        if cache is None or cache.k_pages is None:
            raise ValueError("PagedAttention needs a layer cache with pages")
        n = h.shape[0]
        rows = self.q_dim + (0 if self.shares_kv else 2 * self.kv_dim)
        qkv = ctx.buffer("qkv", (n, rows), ctx.dtype)
        write = cache.writable and not self.shares_kv
        store = (ctx.slots[cache.group], cache.k_pages, cache.v_pages) if write else (None, None, None)
        n_kv = 0 if self.shares_kv else self.n_kv_heads
        pre = isinstance(norm, PreNormed)
        # few rows (decoding): the product's epilogue rotates the heads and writes the cache itself
        tables = None
        if (ctx.dtype == torch.bfloat16 and ctx.fuse_norms and n <= ops.ROPE_PRODUCT_MAX_ROWS
                and self.head_dim % 16 == 0):
            tables = self.position.fuse_spec(ctx, self.head_dim)
        if tables is not None:
            ops.gemm_rope(norm.rows if pre else h, self.wqkv, qkv, self.n_heads, n_kv, self.head_dim, tables[0],
                          tables[1], *store, rms=None if pre else norm, rms_parts=norm.as_gemm_arg() if pre else None)
        else:
            if pre:
                ops.gemm(norm.rows, self.wqkv, qkv, rms_parts=norm.as_gemm_arg())
            else:
                ops.gemm(h, self.wqkv, qkv, rms=norm,
                         workspace=None if norm is not None else split_workspace(ctx, n, rows, self.width))
            self.position.apply_and_store(ctx, qkv, self.n_heads, n_kv, self.head_dim, *store)
        att = ctx.buffer("att", (n, self.q_dim), ctx.dtype)
        paged_attention(ctx, qkv[:, :self.q_dim], att, cache, self.n_heads, self.scale, self.window)
        target, handed_on = emit_target(ctx, n, self.width, self.q_dim, emit, "mixer")
        ops.gemm(att, self.wo, residual, accumulate=True, emit=target,
                 workspace=split_workspace(ctx, n, self.width, self.q_dim))
        return handed_on


class TiedValueAttention(Mixer):
    """Grouped-query attention whose values are its keys: there is no value projection, and a key head as projected
    (bias included, before any norm) is the value head.  Options, each a constructor argument: biases on the query,
    key and output projections; an RMS norm of every query and key head over its dimensions, with a weight for the
    queries and one for the keys that the heads share; the scale of the scores; a window of the last ``window`` keys,
    with the request's first ``keep_first`` keys visible for good.  Positions do not enter the scores.

    Tensors: ``q``, ``k``, ``o`` (and ``q.b``, ``k.b``, ``o.b``; ``q.norm``, ``k.norm``)."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, scale: Optional[float] = None,
                 window: int = 0, keep_first: int = 0, bias: bool = True, qk_norm: bool = True, eps: float = 1e-5):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key heads")
        if keep_first and not window:
            raise ValueError("kept first keys go with a window")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.window, self.keep_first = int(window), int(keep_first)
        self.bias, self.qk_norm, self.eps = bool(bias), bool(qk_norm), float(eps)
        self.q_dim, self.kv_dim = n_heads * head_dim, n_kv_heads * head_dim
        self.cache_spec = CacheSpec(n_kv_heads, head_dim, WINDOW if window > 0 else FULL, self.window, self.keep_first)
        self.wqk = self.wo = self.bias_q = self.bias_k = self.bias_o = self.norm_q = self.norm_k = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {"q": TensorSpec((self.q_dim, self.width)), "k": TensorSpec((self.kv_dim, self.width)),
                 "o": TensorSpec((self.width, self.q_dim))}
        if self.bias:
            specs.update({"q.b": TensorSpec((self.q_dim,), kind="f32", init="normal"),
                          "k.b": TensorSpec((self.kv_dim,), kind="f32", init="normal"),
                          "o.b": TensorSpec((self.width,), kind="f32", init="normal")})
        if self.qk_norm:
            specs.update({"q.norm": TensorSpec((self.head_dim,), kind="f32", init="ones"),
                          "k.norm": TensorSpec((self.head_dim,), kind="f32", init="ones")})
        return specs

    def load(self, tensors):
        self.wqk = torch.cat([tensors["q"], tensors["k"]], 0)   # one product computes both
        self.wo = tensors["o"].contiguous()
        if self.bias:
            self.bias_q, self.bias_k, self.bias_o = (tensors[n].contiguous() for n in ("q.b", "k.b", "o.b"))
        if self.qk_norm:
            self.norm_q, self.norm_k = tensors["q.norm"].contiguous(), tensors["k.norm"].contiguous()

    def streamed_matrices(self):
        return [self.wqk, self.wo]

    def problems(self, dtype, page_size):
        out = []   # (sizes that the matrix-core products do not take go through the plain product)
        if self.head_dim > ops.MAX_HEAD_DIM:
            out.append(("dim", f"{self.head_dim} is above {ops.MAX_HEAD_DIM}, the largest head the attention kernels take"))
        return out

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``; with ``store`` writes them there instead (float32 either way) or leaves
        them in slices, and returns what ``product_in_slices`` does."""
        if cache is None or cache.k_pages is None:
            raise ValueError("TiedValueAttention needs a layer cache with pages")
        n = h.shape[0]
        slots = ctx.slots[cache.group] if cache.writable else None
        if n > ops.ROPE_PRODUCT_MAX_ROWS and slots is not None:
            # many rows: values are written into the rows behind the keys, and the kernel that takes a step's keys and
            # values to their pages in whole lines does the cache write (no rotation)
            rows = ctx.buffer("qkv", (n, self.q_dim + 2 * self.kv_dim), ctx.dtype)
            qk = rows[:, :self.q_dim + self.kv_dim]
            product(ctx, h, self.wqk, qk)
            ops.qk_norm_store(rows, self.bias_q, self.bias_k, self.norm_q, self.norm_k, self.eps, None, None, None,
                              self.n_heads, self.n_kv_heads, self.head_dim, values_in_rows=True)
            ops.rope_store(rows, None, None, slots, cache.k_pages, cache.v_pages, self.n_heads, self.n_kv_heads,
                           self.head_dim, rotate=False, portions=ctx.portions())
        else:
            qk = ctx.buffer("qk", (n, self.q_dim + self.kv_dim), ctx.dtype)
            product(ctx, h, self.wqk, qk)
            ops.qk_norm_store(qk, self.bias_q, self.bias_k, self.norm_q, self.norm_k, self.eps, slots,
                              cache.k_pages if slots is not None else None, cache.v_pages if slots is not None else None,
                              self.n_heads, self.n_kv_heads, self.head_dim)
        att = ctx.buffer("att", (n, self.q_dim), ctx.dtype)
        paged_attention(ctx, qk[:, :self.q_dim], att, cache, self.n_heads, self.scale, self.window, self.keep_first)
        product(ctx, att, self.wo, residual, accumulate=not store)
        if self.bias_o is not None:
            ops.add_bias(residual, self.bias_o)


def cache_head_cols(dim: int, vdim: int) -> int:
    """Columns of a head in the pages of a layer whose keys have ``dim`` channels and whose values have ``vdim``: the
    cache and the attention kernels work on heads of one size, so both are filled up with zeros (which change neither a
    score nor a weighted sum) to the larger of the two, and on to a multiple of 16 where the matrix-core kernels then
    take the head, else to a multiple of 8."""
    most = max(dim, vdim)
    cols = -(-most // 16) * 16
    return cols if cols <= 128 else -(-most // 8) * 8


class ShortConvAttention(Mixer):
    """Grouped-query attention whose projections pass a short causal convolution over time before anything else:
    q, k, v = W h; each channel of the three convolved over its request's tokens with ``taps`` weights (``q.conv`` ...,
    [channels, taps], zeros before the first token; ``taps`` 0: no convolution); the first ``rot_dims`` channels of every
    query and key head turned by the position in neighbouring pairs (2i, 2i + 1), frequencies base^(-2i / rot_dims);
    with ``qk_norm`` every query and key head divided by its root mean square; scores q . k * scale over the last
    ``window`` keys (0: all); softmax; output projection.  Key and value heads may differ in size (``dim``, ``vdim``).

    The request's last taps - 1 projections are its state (``state_spec``), beside the pages of keys and values."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int, scale: Optional[float] = None,
                 window: int = 0, taps: int = 0, rot_dims: int = 0, rot_base: float = 10000.0, qk_norm: bool = True,
                 eps: float = 1e-5):
        from .rotary import Rotary
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key heads")
        if rot_dims % 2 or not 0 <= rot_dims <= dim:
            raise ValueError(f"{rot_dims} rotated channels: an even number up to the key size {dim}")
        self.width, self.n_heads, self.n_kv_heads, self.dim, self.vdim = width, n_heads, n_kv_heads, dim, vdim
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(dim)
        self.window, self.taps, self.rot_dims = int(window), int(taps), int(rot_dims)
        self.qk_norm, self.eps = bool(qk_norm), float(eps)
        self.head_cols = cache_head_cols(dim, vdim)
        self.channels = (n_heads + n_kv_heads) * dim + n_kv_heads * vdim
        self.position = Rotary(rot_dims, rot_base) if rot_dims else None
        self.cache_spec = CacheSpec(n_kv_heads, self.head_cols, WINDOW if window > 0 else FULL, self.window)
        self.state_spec = StateSpec((self.taps - 1, self.channels), torch.float32, 0.0) if self.taps > 1 else None
        self.wqkv = self.wo = self.wconv = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        H, G, D, V = self.n_heads, self.n_kv_heads, self.dim, self.vdim
        specs = {"q": TensorSpec((H * D, self.width)), "k": TensorSpec((G * D, self.width)),
                 "v": TensorSpec((G * V, self.width)), "o": TensorSpec((self.width, H * V))}
        if self.taps:
            specs.update({"q.conv": TensorSpec((H * D, self.taps), kind="f32"), "k.conv": TensorSpec((G * D, self.taps), kind="f32"),
                          "v.conv": TensorSpec((G * V, self.taps), kind="f32")})
        return specs

    def load(self, tensors):
        parts = [tensors["q"], tensors["k"], tensors["v"]]
        if self.channels % 8:   # rows of the product's result then begin at 16-byte words
            parts.append(torch.zeros((8 - self.channels % 8, self.width), dtype=parts[0].dtype, device=parts[0].device))
        self.wqkv = torch.cat(parts, 0)
        # the output projection takes heads of head_cols columns, the columns beyond vdim being zero
        o = tensors["o"]
        wo = torch.zeros((self.width, self.n_heads, self.head_cols), dtype=o.dtype, device=o.device)
        wo[:, :, :self.vdim] = o.view(self.width, self.n_heads, self.vdim)
        self.wo = wo.view(self.width, self.n_heads * self.head_cols)
        if self.taps:
            self.wconv = torch.cat([tensors["q.conv"], tensors["k.conv"], tensors["v.conv"]], 0).float().contiguous()

    def streamed_matrices(self):
        return [self.wqkv, self.wo]

    def problems(self, dtype, page_size):
        out = []
        if self.head_cols > ops.MAX_HEAD_DIM:
            out.append(("dim", f"heads of {max(self.dim, self.vdim)} channels are above {ops.MAX_HEAD_DIM}, the largest head "
                               f"the attention kernels take"))
        if self.taps > ops.CONV_MAX_TAPS:
            out.append(("taps", f"{self.taps} is above {ops.CONV_MAX_TAPS}, the longest convolution the kernel takes"))
        return out

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``; with ``store`` writes them there instead (float32 either way) or leaves
        them in slices, and returns what ``product_in_slices`` does."""
        if cache is None or cache.k_pages is None or (self.taps > 1 and cache.state is None):
            raise ValueError("ShortConvAttention needs a layer cache with pages (and state, with a convolution)")
        n = h.shape[0]
        H, G, hc = self.n_heads, self.n_kv_heads, self.head_cols
        proj = ctx.buffer("conv_proj", (n, self.wqkv.shape[0]), ctx.dtype)
        product(ctx, h, self.wqkv, proj)
        cos, sin = self.position.table(ctx) if self.position is not None else (None, None)
        heads = ctx.buffer("conv_heads", (n, (H + 2 * G) * hc), ctx.dtype)
        slots = ctx.slots[cache.group] if cache.writable else None
        direct = slots is not None and n <= ops.ROPE_PRODUCT_MAX_ROWS
        ops.conv_heads(proj, self.wconv, cache.state, ctx, cos, sin, self.rot_dims, self.eps, self.qk_norm, heads, hc,
                       slots if direct else None, cache.k_pages, cache.v_pages, H, G, self.dim, self.vdim)
        if slots is not None and not direct:
            # many rows: the kernel that takes a step's keys and values to their pages in whole lines
            ops.rope_store(heads, None, None, slots, cache.k_pages, cache.v_pages, H, G, hc, rotate=False,
                           portions=ctx.portions())
        att = ctx.buffer("att", (n, H * hc), ctx.dtype)
        paged_attention(ctx, heads[:, :H * hc], att, cache, H, self.scale, self.window)
        product(ctx, att, self.wo, residual, accumulate=not store)


def _stack_rows(parts, width: int) -> torch.Tensor:
    """Matrices stacked by rows into one product, filled up with zero rows to a multiple of 8 (rows of the product's
    result then begin at 16-byte words)."""
    parts = list(parts)
    rows = sum(p.shape[0] for p in parts)
    if rows % 8:
        parts.append(torch.zeros((8 - rows % 8, width), dtype=parts[0].dtype, device=parts[0].device))
    return torch.cat(parts, 0)


class LatentAttention(Mixer):
    """Attention whose queries, keys and values come through narrow latents.  c_q = norm(W_dq h) (RMS norm with a weight),
    q = W_uq c_q, every query head [dim columns as they are | rot_dim columns that are rotated].  W_dkv h has kv_rank + rot_dim
    rows: the first kv_rank, normed with a weight, are the latent c; the last rot_dim, not normed, are one rotated key part
    that all heads share.  A head's key is [W_uk c | the shared part], its value W_uv c; scores q . k * scale over the last
    ``window`` keys (0: all); softmax.  The first ``rot_dims`` of the rot_dim columns turn with the position in half-split
    pairs (i, i + rot_dims / 2), frequencies base^(-2i / rot_dims).  The heads are multiplied by sigmoid(W_g h) before the
    output projection.

    Tensors: ``dq``, ``dq.norm``, ``uq``, ``dkv``, ``dkv.norm``, ``uk``, ``uv``, ``g``, ``o``.  The pages hold every head's key
    and value as attention reads them (heads of ``cache_head_cols(dim + rot_dim, vdim)`` columns)."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int, kv_rank: int, scale: float,
                 window: int = 0, rot_dims: Optional[int] = None, rot_base: float = 10000.0, eps: float = 1e-5):
        from .rotary import Rotary
        rot_dims = rot_dim if rot_dims is None else rot_dims
        if rot_dims % 2 or not 0 <= rot_dims <= rot_dim:
            raise ValueError(f"{rot_dims} rotated columns: an even number up to rot_dim {rot_dim}")
        self.width, self.n_heads, self.dim, self.rot_dim, self.vdim = width, n_heads, dim, rot_dim, vdim
        self.q_rank, self.kv_rank = q_rank, kv_rank
        self.scale, self.window, self.rot_dims, self.eps = float(scale), int(window), int(rot_dims), float(eps)
        self.head_cols = cache_head_cols(dim + rot_dim, vdim)
        self.position = Rotary(rot_dims, rot_base) if rot_dims else None
        self.cache_spec = CacheSpec(n_heads, self.head_cols, WINDOW if window > 0 else FULL, self.window)
        self.w_in = self.w_uq = self.w_ukv = self.wo = self.norm_q = self.norm_kv = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        H, D, R, V = self.n_heads, self.dim, self.rot_dim, self.vdim
        return {"dq": TensorSpec((self.q_rank, self.width)), "dq.norm": TensorSpec((self.q_rank,), kind="f32", init="ones"),
                "uq": TensorSpec((H * (D + R), self.q_rank)),
                "dkv": TensorSpec((self.kv_rank + R, self.width)), "dkv.norm": TensorSpec((self.kv_rank,), kind="f32", init="ones"),
                "uk": TensorSpec((H * D, self.kv_rank)), "uv": TensorSpec((H * V, self.kv_rank)),
                "g": TensorSpec((H * V, self.width)), "o": TensorSpec((self.width, H * V))}

    def load(self, tensors):
        # one product reads the mixer's input for both latents, the shared key part and the gate
        self.w_in = _stack_rows([tensors["dq"], tensors["dkv"], tensors["g"]], self.width)
        self.w_uq = tensors["uq"].contiguous()
        self.w_ukv = _stack_rows([tensors["uk"], tensors["uv"]], self.kv_rank)
        self.wo = tensors["o"].contiguous()
        self.norm_q, self.norm_kv = tensors["dq.norm"].float().contiguous(), tensors["dkv.norm"].float().contiguous()

    def streamed_matrices(self):
        return [self.w_in, self.w_uq, self.w_ukv, self.wo]

    def problems(self, dtype, page_size):
        if self.head_cols > ops.MAX_HEAD_DIM:
            return [("dim", f"heads of {max(self.dim + self.rot_dim, self.vdim)} columns are above {ops.MAX_HEAD_DIM}, the "
                            f"largest head the attention kernels take")]
        return []

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``; with ``store`` writes them there instead (float32 either way) or leaves
        them in slices, and returns what ``product_in_slices`` does."""
        if cache is None or cache.k_pages is None:
            raise ValueError("LatentAttention needs a layer cache with pages")
        n = h.shape[0]
        H, D, R, V, hc = self.n_heads, self.dim, self.rot_dim, self.vdim, self.head_cols
        first = ctx.buffer("latent_in", (n, self.w_in.shape[0]), ctx.dtype)     # [c_q | c | shared key part | gate]
        product(ctx, h, self.w_in, first)
        c_q = ctx.buffer("latent_cq", (n, self.q_rank), ctx.dtype)
        c_kv = ctx.buffer("latent_ckv", (n, self.kv_rank), ctx.dtype)
        ops.norm_slices(first, self.eps, (0, self.norm_q, c_q), (self.q_rank, self.norm_kv, c_kv))
        q = ctx.buffer("latent_q", (n, self.w_uq.shape[0]), ctx.dtype)
        product(ctx, c_q, self.w_uq, q)
        kv = ctx.buffer("latent_kv", (n, self.w_ukv.shape[0]), ctx.dtype)
        product(ctx, c_kv, self.w_ukv, kv)
        cos, sin = self.position.table(ctx) if self.position is not None else (None, None)
        heads = ctx.buffer("latent_heads", (n, 3 * H * hc), ctx.dtype)
        slots = ctx.slots[cache.group] if cache.writable else None
        direct = slots is not None and n <= ops.ROPE_PRODUCT_MAX_ROWS
        shared = self.q_rank + self.kv_rank
        ops.latent_heads(q, kv, first[:, shared:shared + max(R, 1)], cos, sin, self.rot_dims, heads, hc,
                         slots if direct else None, cache.k_pages, cache.v_pages, H, D, R, V)
        if slots is not None and not direct:
            # many rows: the kernel that takes a step's keys and values to their pages in whole lines
            ops.rope_store(heads, None, None, slots, cache.k_pages, cache.v_pages, H, H, hc, rotate=False,
                           portions=ctx.portions())
        att = ctx.buffer("att", (n, H * hc), ctx.dtype)
        paged_attention(ctx, heads[:, :H * hc], att, cache, H, self.scale, self.window)
        gated = ctx.buffer("latent_gated", (n, H * V), ctx.dtype)
        ops.gate_heads(att, hc, first[:, shared + R:shared + R + H * V], gated, H, V)
        if store:   # the caller's norm adds the slices of a product that divides k
            return product_in_slices(ctx, gated, self.wo, residual)
        product(ctx, gated, self.wo, residual, accumulate=True)
        return None


class DifferentialAttention(Mixer):
    """Grouped-query attention with two softmax maps a head over the same values: every query and key head holds two
    maps of ``dim`` columns, [map 1 | map 2]; each map is divided by its root mean square and multiplied by a weight of
    dim numbers (``q.norm``, ``k.norm``, shared by all heads and maps); query maps are also multiplied by the
    temperature 1 + coef * ln(floor((position + 1) / every) + 1) (``temp_every`` 0: not); scores q . k * scale over all
    earlier keys; positions enter nowhere else.  With a1, a2 the maps' outputs, o = a1 - lambda a2, lambda =
    exp(lq1 . lk1) - exp(lq2 . lk2) + diff (one number for the layer), then o / sqrt(mean(o^2) + eps) * (1 - diff) over
    the head's vdim values, and the output projection.

    The two maps of a head are run as two query heads of 2 dim columns, [q1 | 0] and [0 | q2], over one key head
    [k1 | k2]: the zeros leave each map its own score, and both read the same cached values.

    Tensors: ``q``, ``k``, ``v``, ``q.norm``, ``k.norm``, ``lq1``, ``lk1``, ``lq2``, ``lk2``, ``o``."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int, scale: float, diff: float,
                 temp_coef: float = 0.0, temp_every: int = 0, eps: float = 1e-5):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key heads")
        self.width, self.n_heads, self.n_kv_heads, self.dim, self.vdim = width, n_heads, n_kv_heads, dim, vdim
        self.scale, self.diff, self.eps = float(scale), float(diff), float(eps)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        self.head_cols = cache_head_cols(2 * dim, vdim)
        self.cache_spec = CacheSpec(n_kv_heads, self.head_cols, FULL, 0)
        self.wqkv = self.wo = self.norm_q = self.norm_k = self.lam = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        H, G, D, V = self.n_heads, self.n_kv_heads, self.dim, self.vdim
        specs = {"q": TensorSpec((H * 2 * D, self.width)), "k": TensorSpec((G * 2 * D, self.width)),
                 "v": TensorSpec((G * V, self.width)), "o": TensorSpec((self.width, H * V)),
                 "q.norm": TensorSpec((D,), kind="f32", init="ones"), "k.norm": TensorSpec((D,), kind="f32", init="ones")}
        for name in ("lq1", "lk1", "lq2", "lk2"):
            specs[name] = TensorSpec((D,), kind="f32")
        return specs

    def load(self, tensors):
        self.wqkv = _stack_rows([tensors["q"], tensors["k"], tensors["v"]], self.width)
        self.wo = tensors["o"].contiguous()
        self.norm_q, self.norm_k = tensors["q.norm"].float().contiguous(), tensors["k.norm"].float().contiguous()
        one, two = (tensors["lq1"].float() * tensors["lk1"].float()).sum(), (tensors["lq2"].float() * tensors["lk2"].float()).sum()
        self.lam = (torch.exp(one) - torch.exp(two) + self.diff).reshape(1).contiguous()   # a number of the weights alone

    def streamed_matrices(self):
        return [self.wqkv, self.wo]

    def problems(self, dtype, page_size):
        if self.head_cols > ops.MAX_HEAD_DIM:
            return [("dim", f"heads of {max(2 * self.dim, self.vdim)} columns (two maps of dim) are above {ops.MAX_HEAD_DIM}, "
                            f"the largest head the attention kernels take")]
        return []

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``; with ``store`` writes them there instead (float32 either way) or leaves
        them in slices, and returns what ``product_in_slices`` does."""
        if cache is None or cache.k_pages is None:
            raise ValueError("DifferentialAttention needs a layer cache with pages")
        n = h.shape[0]
        H, G, V, hc = self.n_heads, self.n_kv_heads, self.vdim, self.head_cols
        proj = ctx.buffer("diff_proj", (n, self.wqkv.shape[0]), ctx.dtype)
        product(ctx, h, self.wqkv, proj)
        heads = ctx.buffer("diff_heads", (n, (2 * H + 2 * G) * hc), ctx.dtype)
        slots = ctx.slots[cache.group] if cache.writable else None
        direct = slots is not None and n <= ops.ROPE_PRODUCT_MAX_ROWS
        ops.diff_heads(proj, self.norm_q, self.norm_k, self.eps, self.temp_coef, self.temp_every, ctx.positions, heads, hc,
                       slots if direct else None, cache.k_pages, cache.v_pages, H, G, self.dim, V)
        if slots is not None and not direct:
            ops.rope_store(heads, None, None, slots, cache.k_pages, cache.v_pages, 2 * H, G, hc, rotate=False,
                           portions=ctx.portions())
        # the two maps' results stay 32-bit until their difference is taken (where they are close, rounding each
        # first would be most of what is left), wherever the attention kernels write such rows
        wide = ctx.dtype == torch.bfloat16 and ctx.tuned and ops.tuned_attention_supports(cache.k_pages, 2 * H, 0, 0)
        att = ctx.buffer("att32", (n, 2 * H * hc), torch.float32) if wide else ctx.buffer("att", (n, 2 * H * hc), ctx.dtype)
        paged_attention(ctx, heads[:, :2 * H * hc], att, cache, 2 * H, self.scale, 0)
        o = ctx.buffer("diff_o", (n, H * V), ctx.dtype)
        ops.diff_combine(att, hc, self.lam, 1.0 - self.diff, self.eps, o, H, V)
        if store:   # the caller's norm adds the slices of a product that divides k
            return product_in_slices(ctx, o, self.wo, residual)
        product(ctx, o, self.wo, residual, accumulate=True)
        return None


class GatedAttention(Mixer):
    """Grouped-query attention whose heads are gated before the output projection, with a sink in the softmax, and whose
    query and key heads are prepared in one pass.  Every option is a constructor argument:

    * ``bias``: biases on the query, key and value projections (``q.b``, ``k.b``, ``v.b``);
    * ``taps`` > 0: a short causal convolution over time on every query and key channel right after the projection
      (``q.conv``, ``k.conv`` [channels, taps], zeros before the request's first token); the request's last taps - 1
      projections are its state;
    * ``tied_values``: no value projection: the key channels as they leave the convolution are the value heads;
    * ``qk_norm``: "joint": one RMS norm over all query channels (and one over all key channels) before they are cut into
      heads, a weight a channel (``q.norm`` [heads * dim]); "head": every head over its ``dim`` channels with ``dim``
      weights that the heads share;
    * the first ``rot_dims`` channels of every query and key head turn with the position: ``rot_pairs`` "neighbours"
      (channel 2i with 2i + 1) or "halves" (i with i + rot_dims / 2), frequencies base^(-2i / rot_dims), with
      ``rot_scaling = (factor, original, fast, slow)`` stretched as ``parts.rotary.Rotary`` says;
    * scores q . k * ``scale``, with ``softcap`` > 0 then softcap * tanh(score / softcap); ``chunk`` > 0: a token sees the
      keys of its own run of ``chunk`` positions (runs counted from the request's first token), else all earlier keys;
    * ``sink``: "zero": one is added to the softmax's denominator (a sink of score 0); "learned": exp(sink_h), one number a
      head (``sink``); None: a plain softmax;
    * ``gate``: "head": head h times sigmoid(W_g h)_h (``g`` [heads, width]); "channel": every channel of the heads times
      its own sigmoid (``g`` [heads * vdim, width]); the gate reads the mixer's input;
    * the output projection ``o`` on the gated heads.

    One product makes queries, keys, values and gates; ``ops.qk_heads`` prepares the heads (and writes the cache in steps
    of few rows); the framework's paged attention kernels do the rest."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int, scale: float, eps: float,
                 bias: bool = False, taps: int = 0, tied_values: bool = False, qk_norm: str = "head", rot_dims: int = 0,
                 rot_base: float = 10000.0, rot_pairs: str = "halves", rot_scaling=None, softcap: float = 0.0, chunk: int = 0,
                 sink: Optional[str] = None, gate: str = "channel"):
        from .rotary import Rotary
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key heads")
        if rot_dims % 2 or not 0 <= rot_dims <= dim:
            raise ValueError(f"{rot_dims} rotated channels: an even number up to the key size {dim}")
        if tied_values and vdim != dim:
            raise ValueError(f"values that are the keys have the keys' size: dim {dim}, vdim {vdim}")
        if qk_norm == "joint" and taps:
            raise ValueError("one norm over all of q (and of k) behind a convolution is not served: qk_norm='head' goes with taps")
        if qk_norm not in ("joint", "head") or rot_pairs not in ("neighbours", "halves") or sink not in (None, "zero", "learned") \
                or gate not in ("head", "channel"):
            raise ValueError("qk_norm: joint | head; rot_pairs: neighbours | halves; sink: None | zero | learned; gate: head | channel")
        self.width, self.n_heads, self.n_kv_heads, self.dim, self.vdim = width, n_heads, n_kv_heads, dim, vdim
        self.scale, self.eps, self.bias, self.taps, self.tied_values = float(scale), float(eps), bool(bias), int(taps), bool(tied_values)
        self.qk_norm, self.rot_dims, self.rot_pairs, self.softcap, self.chunk = qk_norm, int(rot_dims), rot_pairs, float(softcap), int(chunk)
        self.sink, self.gate = sink, gate
        self.head_cols = cache_head_cols(dim, vdim)
        self.channels = (n_heads + n_kv_heads) * dim
        self.value_cols = 0 if tied_values else n_kv_heads * vdim
        self.gate_cols = n_heads if gate == "head" else n_heads * vdim
        self.position = Rotary(rot_dims, rot_base, rot_scaling) if rot_dims else None
        # (the pages of a run that has ended are given back: no later token reads them)
        self.cache_spec = CacheSpec(n_kv_heads, self.head_cols, RUNS if self.chunk else FULL, self.chunk)
        self.state_spec = StateSpec((self.taps - 1, self.channels), torch.float32, 0.0) if self.taps > 1 else None
        self.w_in = self.wo = self.b_in = self.wconv = self.norm_q = self.norm_k = self.sinks = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        H, G, D, V = self.n_heads, self.n_kv_heads, self.dim, self.vdim
        specs = {"q": TensorSpec((H * D, self.width)), "k": TensorSpec((G * D, self.width))}
        if not self.tied_values:
            specs["v"] = TensorSpec((G * V, self.width))
        if self.bias:
            specs["q.b"] = TensorSpec((H * D,), kind="f32")
            specs["k.b"] = TensorSpec((G * D,), kind="f32")
            if not self.tied_values:
                specs["v.b"] = TensorSpec((G * V,), kind="f32")
        joint = self.qk_norm == "joint"
        specs["q.norm"] = TensorSpec((H * D if joint else D,), kind="f32", init="ones")
        specs["k.norm"] = TensorSpec((G * D if joint else D,), kind="f32", init="ones")
        if self.taps:
            specs["q.conv"] = TensorSpec((H * D, self.taps), kind="f32")
            specs["k.conv"] = TensorSpec((G * D, self.taps), kind="f32")
        if self.sink == "learned":
            specs["sink"] = TensorSpec((H,), kind="f32")
        specs["g"] = TensorSpec((self.gate_cols, self.width))
        specs["o"] = TensorSpec((self.width, H * V))
        return specs

    def load(self, tensors):
        parts = [tensors["q"], tensors["k"]] + ([] if self.tied_values else [tensors["v"]]) + [tensors["g"]]
        self.w_in = _stack_rows(parts, self.width)   # one product reads the mixer's input for all of them
        self.wo = tensors["o"].contiguous()
        if self.bias:
            self.b_in = torch.cat([tensors["q.b"], tensors["k.b"]] + ([] if self.tied_values else [tensors["v.b"]])).float().contiguous()
        self.norm_q, self.norm_k = tensors["q.norm"].float().contiguous(), tensors["k.norm"].float().contiguous()
        if self.taps:
            # a row a tap: neighbouring channels' weights of one tap lie side by side
            self.wconv = torch.cat([tensors["q.conv"], tensors["k.conv"]], 0).float().t().contiguous()
        if self.sink == "learned":
            self.sinks = tensors["sink"].float().contiguous()
        elif self.sink == "zero":
            self.sinks = torch.zeros(self.n_heads, dtype=torch.float32, device=self.wo.device)

    def streamed_matrices(self):
        return [self.w_in, self.wo]

    def problems(self, dtype, page_size):
        out = []
        if self.head_cols > ops.MAX_HEAD_DIM:
            out.append(("dim", f"heads of {max(self.dim, self.vdim)} channels are above {ops.MAX_HEAD_DIM}, the largest head "
                               f"the attention kernels take"))
        if self.taps > ops.CONV_MAX_TAPS:
            out.append(("taps", f"{self.taps} is above {ops.CONV_MAX_TAPS}, the longest convolution the kernel takes"))
        return out

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``; with ``store`` writes them there instead (float32 either way) or leaves
        them in slices, and returns what ``product_in_slices`` does."""
        if cache is None or cache.k_pages is None or (self.taps > 1 and cache.state is None):
            raise ValueError("GatedAttention needs a layer cache with pages (and state, with a convolution)")
        n = h.shape[0]
        H, G, V, hc = self.n_heads, self.n_kv_heads, self.vdim, self.head_cols
        proj = ctx.buffer("gated_proj", (n, self.w_in.shape[0]), ctx.dtype)   # [q | k | v | gate]
        product(ctx, h, self.w_in, proj)
        cos, sin = self.position.table(ctx) if self.position is not None else (None, None)
        heads = ctx.buffer("gated_heads", (n, (H + 2 * G) * hc), ctx.dtype)
        slots = ctx.slots[cache.group] if cache.writable else None
        direct = slots is not None and n <= ops.ROPE_PRODUCT_MAX_ROWS
        ops.qk_heads(proj, ctx, heads, hc, H, G, self.dim, V, self.eps, self.qk_norm == "joint", self.norm_q, self.norm_k,
                     bias=self.b_in, wconv=self.wconv, state=cache.state if self.taps > 1 else None, cos=cos, sin=sin,
                     rot=self.rot_dims, magnitude=self.position.magnitude if self.position is not None else 1.0,
                     neighbours=self.rot_pairs == "neighbours", tied=self.tied_values, slots=slots if direct else None,
                     k_pages=cache.k_pages, v_pages=cache.v_pages)
        if slots is not None and not direct:
            # many rows: the kernel that takes a step's keys and values to their pages in whole lines
            ops.rope_store(heads, None, None, slots, cache.k_pages, cache.v_pages, H, G, hc, rotate=False,
                           portions=ctx.portions())
        att = ctx.buffer("att", (n, H * hc), ctx.dtype)
        paged_attention(ctx, heads[:, :H * hc], att, cache, H, self.scale, 0, 0, self.chunk, self.softcap, self.sinks)
        gated = ctx.buffer("gated_rows", (n, H * V), ctx.dtype)
        at = self.channels + self.value_cols
        ops.gate_rows(att, hc, proj[:, at:at + self.gate_cols], gated, H, V, self.gate == "head")
        if store:   # the caller's pass over the rows adds the slices of a product that divides k
            return product_in_slices(ctx, gated, self.wo, residual)
        product(ctx, gated, self.wo, residual, accumulate=True)
        return None
