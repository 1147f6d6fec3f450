"""A feed-forward made of many narrow gated units (experts), a few of them picked anew for every token.

z = W_router h in 32-bit and s = sigmoid(z).  A token's experts are the ``top`` largest of s + correction (the correction
takes part in the picking alone); expert e of them gets the weight a_e = scale * s_e / (1e-20 + sum of the picked s).  An
expert computes y_e = W_down (silu(W_gate h) * (W_up h)), no biases, and the token's result is sum_e a_e y_e.  With
``shared_ff`` one more such unit serves all tokens, its result scaled by sigmoid(W_sg h), a scalar per token.

The experts' gate matrices are stacked by rows, then their up matrices, then the shared expert's gate and up; the down
matrices stand side by side, the shared expert's last.  A step of few tokens runs every expert on every token: one
product gives every expert's gate and up sums; the unit's kernel multiplies each expert's columns by the token's weight
for it, zero for an expert that was not chosen; one product with the down matrices then adds up exactly the chosen
experts' outputs, and every matrix is read once.  A step of many tokens (``routed``) runs an expert on the tokens that
chose it alone: the (token, choice) entries are put in the order of their experts on the device, the two products go
over row tiles that lie in one expert each, and each token's chosen rows are added up with their weights.

Other routers and units are options of the same part: ``scoring="softmax"`` (s = softmax(z) over all experts);
``renorm=False`` (a_e = scale * s_e as it stands); ``groups=(count, keep)`` (the experts form ``count`` equal runs of
neighbours, and only experts of the ``keep`` runs whose best s + correction is largest can be chosen);
``unit="relu2"`` (an expert is W_down relu(W_up h)^2: one matrix in, no gate half); ``shared_gate=False`` (the shared
expert's result is added as it is).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import FeedForward, TensorSpec, product, split_workspace


class RoutedExperts(FeedForward):
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_experts: int, top: int, expert_ff: int, router_scale: float = 1.0,
                 shared_ff: int = 0, correction: bool = True, scoring: str = "sigmoid", renorm: bool = True,
                 groups=None, unit: str = "swiglu", shared_gate: bool = True):
        if not 1 <= top <= n_experts:
            raise ValueError(f"{top} experts a token out of {n_experts}")
        if scoring not in ("sigmoid", "softmax") or unit not in ("swiglu", "relu2"):
            raise ValueError("scoring: sigmoid | softmax; unit: swiglu | relu2")
        self.width, self.n_experts, self.top, self.expert_ff = width, int(n_experts), int(top), int(expert_ff)
        self.router_scale, self.shared_ff, self.has_correction = float(router_scale), int(shared_ff), bool(correction)
        self.scoring, self.renorm, self.unit, self.shared_gate = scoring, bool(renorm), unit, bool(shared_gate)
        self.groups = None if not groups else (int(groups[0]), int(groups[1]))
        if self.groups is not None:
            count, keep = self.groups
            if count < 1 or n_experts % count or not 1 <= keep <= count or keep * (n_experts // count) < top:
                raise ValueError(f"{n_experts} experts in {count} groups of which {keep} are kept, {top} experts a token")
        self.inter = self.n_experts * self.expert_ff + self.shared_ff
        self.halves = 2 if unit == "swiglu" else 1      # matrices on the way in: gate and up, or up alone
        self.w_router = self.correction = self.w_gate_up = self.w_down = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        ins = ("gate", "up") if self.unit == "swiglu" else ("up",)
        for e in range(self.n_experts):
            for m in ins:
                specs[f"e{e}.{m}"] = TensorSpec((self.expert_ff, self.width))
            specs[f"e{e}.down"] = TensorSpec((self.width, self.expert_ff))
        specs["router"] = TensorSpec((self.n_experts, self.width))
        if self.has_correction:
            specs["correction"] = TensorSpec((self.n_experts,), kind="f32", init="normal")
        if self.shared_ff:
            for m in ins:
                specs[f"shared.{m}"] = TensorSpec((self.shared_ff, self.width))
            specs["shared.down"] = TensorSpec((self.width, self.shared_ff))
            if self.shared_gate:
                specs["shared.sg"] = TensorSpec((1, self.width))
        return specs

    def load(self, tensors):
        names = [f"e{e}" for e in range(self.n_experts)]
        shared = ["shared"] if self.shared_ff else []
        ins = ("gate", "up") if self.unit == "swiglu" else ("up",)
        # every expert's gate rows, then their up rows, then the shared expert's gate and up rows (with one matrix in: the
        # experts' up rows, then the shared expert's)
        self.w_gate_up = torch.cat([tensors[f"{n}.{m}"] for m in ins for n in names] +
                                   [tensors[f"shared.{m}"] for m in ins if self.shared_ff], 0)
        self.w_down = torch.cat([tensors[f"{n}.down"] for n in names + shared], 1).contiguous()
        router = [tensors["router"]] + ([tensors["shared.sg"]] if self.shared_ff and self.shared_gate else [])
        self.w_router = torch.cat(router, 0).contiguous()
        self.correction = tensors["correction"].contiguous() if self.has_correction else None

    def streamed_matrices(self):
        return [self.w_router, self.w_gate_up, self.w_down]

    def problems(self, dtype, page_size):
        out = []
        if self.n_experts > ops.MOE_MAX_EXPERTS:
            out.append(("n_experts", f"{self.n_experts} is above {ops.MOE_MAX_EXPERTS}, the most experts the router's kernel takes"))
        if self.top > ops.MOE_MAX_TOP:
            out.append(("top", f"{self.top} is above {ops.MOE_MAX_TOP}, the most experts a token the router's kernel takes"))
        return out

    def forward(self, ctx, h, residual, store: bool = False):
        n, E = h.shape[0], self.n_experts
        cols = E + (1 if self.shared_ff else 0)
        z = ctx.buffer("moe_z", (n, self.w_router.shape[0]), torch.float32)
        product(ctx, h, self.w_router, z)
        combine = ctx.buffer("moe_combine", (n, cols), torch.float32)
        ids = ctx.buffer("moe_ids", (n, self.top), torch.int32)
        weights = ctx.buffer("moe_weights", (n, self.top), torch.float32)
        shared = False if not self.shared_ff else True if self.shared_gate else "whole"
        count, keep = self.groups if self.groups is not None else (0, 0)
        ops.moe_route(z, E, self.correction, self.top, self.router_scale, shared, combine, ids, weights,
                      softmax=self.scoring == "softmax", renorm=self.renorm, groups=count, keep_groups=keep)
        if self.routed(ctx, n):
            return self._routed(ctx, h, residual, store, combine, ids, weights)
        gate_up = ctx.buffer("moe_gate_up", (n, self.halves * self.inter), torch.float32)
        product(ctx, h, self.w_gate_up, gate_up)
        act = ctx.buffer("act", (n, self.inter), ctx.dtype)
        if self.unit == "swiglu":
            ops.moe_gated_units(gate_up, combine, act, E, self.expert_ff)
        else:
            ops.moe_relu2_units(gate_up, combine, act, E, self.expert_ff)
        product(ctx, act, self.w_down, residual, accumulate=not store)
        return None

    def routed(self, ctx, n: int) -> bool:
        """Whether a step of n tokens runs the experts on their own tokens: where the sorted rows, every expert's last
        tile of 64 filled up, are fewer than n rows for every expert, and the matrix-core products take the sizes."""
        E, ff, d = self.n_experts, self.expert_ff, self.width
        return (ctx.dtype == torch.bfloat16 and n > 64 and n * self.top + 64 * E < n * E
                and d % 8 == 0 and ff % 8 == 0 and self.shared_ff % 8 == 0 and self.w_gate_up.data_ptr() % 16 == 0
                and self.w_down.data_ptr() % 16 == 0)

    def _routed(self, ctx, h, residual, store, combine, ids, weights):
        n, E, ff, d, top = h.shape[0], self.n_experts, self.expert_ff, self.width, self.top
        entries = n * top
        tile_rows = 128 if entries >= 256 * E else 64
        tiles = ops.moe_sort_tiles(entries, E, tile_rows)
        counts = ctx.buffer("moe_counts", (E,), torch.int32)
        rows = ctx.buffer("moe_rows", (entries,), torch.int32)
        pos = ctx.buffer("moe_pos", (n, top), torch.int32)
        tile_map = ctx.buffer("moe_tiles", (tiles, 3), torch.int32)
        ops.moe_sort(ids, E, tile_rows, counts, rows, pos, tile_map)
        act = ctx.buffer("act", (entries, ff), torch.bfloat16)
        if self.unit == "swiglu":
            ops.gemm_grouped(h, rows, self.w_gate_up, ff * self.w_gate_up.stride(0), 2 * ff, tile_map, tile_rows, act,
                             silu_mul=True, up_offset=E * ff)
        else:   # the unit in a pass of its own over the experts' rows, in place
            ops.gemm_grouped(h, rows, self.w_gate_up, ff * self.w_gate_up.stride(0), ff, tile_map, tile_rows, act)
            ops.moe_relu2_units(act, None, act, 0, ff)
        y = ctx.buffer("moe_y", (entries, d), torch.float32)
        ops.gemm_grouped(act, None, self.w_down, ff, d, tile_map, tile_rows, y)
        y_shared = gates = None
        if self.shared_ff:
            act_shared = ctx.buffer("moe_act_shared", (n, self.shared_ff), torch.bfloat16)
            w = self.w_gate_up[self.halves * E * ff:]
            if self.unit == "swiglu":
                ops.gemm(h, w, act_shared, silu_mul=True, workspace=split_workspace(ctx, n, 2 * self.shared_ff, d))
            else:
                ops.gemm(h, w, act_shared, workspace=split_workspace(ctx, n, self.shared_ff, d))
                ops.moe_relu2_units(act_shared, None, act_shared, 0, self.shared_ff)
            y_shared = ctx.buffer("moe_y_shared", (n, d), torch.float32)
            w = self.w_down[:, E * ff:]
            ops.gemm(act_shared, w, y_shared, workspace=split_workspace(ctx, n, d, self.shared_ff))
            gates = combine[:, E]
        ops.moe_combine(y, pos, weights, y_shared, gates, residual, accumulate=not store)
        return None
