"""Plain, slow implementation of the Tekilix decoder: whole sequences, no cache, no state carried between calls.

One function per mechanism, float64 throughout, sharing no code with the engine.  ``cfg`` is the parsed
``config.json`` as it stands (nested), ``w`` maps the checkpoint's tensor names to tensors.

Notation: T tokens at positions 0..T-1; H query heads, G key/value heads (query head h reads key/value head
h // (H/G)); dk key size, dv value size per head; a linear weight W is stored [out, in] and applied as x W^T.

A layer:  x <- x + n1b(mixer(n1(x)));  x <- x + n2b(ff(n2(x))), every n a bounded norm  tanh(alpha x) * w + b  with one
number alpha, which needs no statistic of the row.  ``forward(..., coarse=True)`` rounds the activations to bfloat16
where a bfloat16 engine may: how far that moves a position's logits is the scale of the device tests' bfloat16 tolerance.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

from .llama import read_safetensors

F64 = torch.float64


def load_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    w = {k: v.to(F64) for k, v in read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


def exact(x: torch.Tensor) -> torch.Tensor:
    return x


def bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(F64)


# ---------------------------------------------------------------------------------------------- norms
def tanh_norm(w, name: str, x: torch.Tensor) -> torch.Tensor:
    """tanh(alpha x) * weight + bias; alpha a single number."""
    return torch.tanh(w[name + ".alpha"].reshape(()) * x) * w[name] + w[name + ".b"]


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


# ---------------------------------------------------------------------------------------------- positions
def inverse_frequencies(rot: dict) -> torch.Tensor:
    """f_i = base^(-2i / R), i < R/2; with ``scaling`` the slow turns are slowed further: a ramp over i between the
    indices whose period meets ``original / fast`` and ``original / slow`` blends f_i / factor in."""
    R, base = rot["dims"], float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / R) for i in range(R // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f

    def index_of(turns: float) -> float:
        return R * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(sc["fast"])), 0)
    hi = min(math.ceil(index_of(sc["slow"])), R - 1)
    i = torch.arange(R // 2, dtype=F64)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp)


def magnitude(rot: dict) -> float:
    """What cosine and sine are multiplied by: 1 without scaling."""
    sc = rot.get("scaling")
    return 0.1 * math.log(sc["factor"]) + 1.0 if sc else 1.0


def turn(u, v, ang, mag):
    cs, sn = torch.cos(ang) * mag, torch.sin(ang) * mag
    return u * cs - v * sn, v * cs + u * sn


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: Optional[dict], neighbours: bool) -> torch.Tensor:
    """x [T, heads, d]: the first R = rot["dims"] channels of every head turn by angle p f_i, the rest pass.
    ``neighbours``: channel 2i pairs with 2i + 1; else channel i with i + R/2."""
    if not rot or not rot.get("dims"):
        return x
    R = rot["dims"]
    ang = positions.to(F64)[:, None] * inverse_frequencies(rot)[None, :]       # [T, R/2]
    ang = ang[:, None, :]
    mag = magnitude(rot)
    out = x.clone()
    if neighbours:
        a, b = turn(x[..., 0:R:2], x[..., 1:R:2], ang, mag)
        out[..., 0:R:2], out[..., 1:R:2] = a, b
    else:
        a, b = turn(x[..., :R // 2], x[..., R // 2:R], ang, mag)
        out[..., :R // 2], out[..., R // 2:R] = a, b
    return out


# ---------------------------------------------------------------------------------------------- short convolution
def causal_conv(u: torch.Tensor, taps_w: torch.Tensor) -> torch.Tensor:
    """u [T, C], taps_w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the first token."""
    T, C = u.shape
    taps = taps_w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += taps_w[:, j] * u[s]
    return y


# ---------------------------------------------------------------------------------------------- attention
def visible(T: int, chunk: int = 0) -> torch.Tensor:
    """[T, T] truth values: query i sees key j if j <= i and, with chunks, both lie in the same run of ``chunk``
    positions counted from 0."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if chunk:
        ok = ok & (i // chunk == j // chunk)
    return ok


def capped(s: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(s / cap) if cap else s


def softmax_with_sink(s: torch.Tensor, mask: torch.Tensor, sink: torch.Tensor) -> torch.Tensor:
    """s [H, T, T], sink [H]: p_ij = exp(s_ij) / (exp(sink_h) + sum over visible j' of exp(s_ij')).  The sink has
    no value, so the weights of a row sum to less than one."""
    s = s.masked_fill(~mask[None], float("-inf"))
    top = torch.maximum(s.max(-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(s - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink[:, None, None] - top))


def attend(q, k, v, scale: float, cap: float, mask, sink) -> torch.Tensor:
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] -> [T, H, dv]."""
    group = q.shape[1] // k.shape[1]
    kh, vh = k.repeat_interleave(group, 1), v.repeat_interleave(group, 1)
    s = capped(torch.einsum("ihd,jhd->hij", q, kh) * scale, cap)
    return torch.einsum("hij,jhd->ihd", softmax_with_sink(s, mask, sink), vh)


def attention_heads(w, pre: str, m: dict, eps: float, h: torch.Tensor, rnd=exact, positions=None):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] of the mixer ``attention`` as its scores and sums read them."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T) if positions is None else positions
    q = rnd(h @ w[pre + "q"].T + w[pre + "q.b"])
    k = rnd(h @ w[pre + "k"].T + w[pre + "k.b"])
    v = rnd(h @ w[pre + "v"].T + w[pre + "v.b"]).view(T, G, dv)
    q = (unit_rms(q, eps) * w[pre + "q.norm"]).view(T, H, dk)
    k = (unit_rms(k, eps) * w[pre + "k.norm"]).view(T, G, dk)
    return rnd(rotate(q, pos, m.get("rot"), True)), rnd(rotate(k, pos, m.get("rot"), True)), v


def attention(w, pre: str, m: dict, eps: float, h: torch.Tensor, rnd=exact) -> torch.Tensor:
    """Biased projections; one RMS norm over all of q (and of k) before the heads are cut; neighbouring pairs turn;
    capped scores; a sink of score 0; one sigmoid gate a head."""
    T = h.shape[0]
    H, dv = m["heads"], m["vdim"]
    q, k, v = attention_heads(w, pre, m, eps, h, rnd)
    chunk = (m.get("mask") or {"size": 0})["size"]
    o = attend(q, k, v, m["scale"], m.get("softcap") or 0.0, visible(T, chunk), torch.zeros(H, dtype=F64))
    gate = torch.sigmoid(rnd(h @ w[pre + "g"].T))                 # [T, H]
    return rnd((o * gate[:, :, None]).reshape(T, H * dv)) @ w[pre + "o"].T


def attention_2_heads(w, pre: str, m: dict, eps: float, h: torch.Tensor, rnd=exact):
    """q [T, H, dk], k [T, G, dk], v [T, G, dk] of the mixer ``attention_2`` (whole sequences from position 0)."""
    T = h.shape[0]
    H, G, dk = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(T)
    q, k = rnd(h @ w[pre + "q"].T), rnd(h @ w[pre + "k"].T)
    if m.get("conv"):
        q, k = causal_conv(q, w[pre + "q.conv"]), causal_conv(k, w[pre + "k.conv"])
    v = rnd(k).view(T, G, dk)
    q = unit_rms(q.view(T, H, dk), eps) * w[pre + "q.norm"]
    k = unit_rms(k.view(T, G, dk), eps) * w[pre + "k.norm"]
    return rnd(rotate(q, pos, m.get("rot"), False)), rnd(rotate(k, pos, m.get("rot"), False)), v


def attention_2(w, pre: str, m: dict, eps: float, h: torch.Tensor, rnd=exact) -> torch.Tensor:
    """No biases; q and k pass a short convolution over time; the values are the convolved keys; an RMS norm of every
    head with one weight for all heads; halves of the rotated channels pair up; a learned sink a head; a sigmoid gate
    on every channel of the heads."""
    T = h.shape[0]
    H, dk = m["heads"], m["dim"]
    q, k, v = attention_2_heads(w, pre, m, eps, h, rnd)
    chunk = (m.get("mask") or {"size": 0})["size"]
    o = attend(q, k, v, m["scale"], 0.0, visible(T, chunk), w[pre + "sink"])
    gate = torch.sigmoid(rnd(h @ w[pre + "g"].T))            # [T, H dk]
    return rnd(o.reshape(T, H * dk) * gate) @ w[pre + "o"].T


# ---------------------------------------------------------------------------------------------- feed-forward
def squared_relu_unit(w, pre: str, x: torch.Tensor, rnd=exact) -> torch.Tensor:
    z = rnd(x @ w[pre + "up"].T)
    return rnd(torch.relu(z) ** 2) @ w[pre + "down"].T


def route(z: torch.Tensor, correction: torch.Tensor, top: int, groups: Optional[dict]):
    """z [T, E] -> (ids [T, top], weights [T, top]).  s = softmax(z); an expert is picked by s + correction, and only
    out of the ``keep`` groups (of ``count`` runs of neighbouring experts) whose best pick score is largest; its weight
    is s itself, as it stands."""
    s = torch.softmax(z, -1)
    pick = s + correction
    T, E = z.shape
    if groups:
        size = E // groups["count"]
        best = pick.view(T, groups["count"], size).max(-1).values
        kept = torch.zeros(T, groups["count"], dtype=torch.bool)
        kept.scatter_(1, torch.topk(best, groups["keep"], dim=-1).indices, True)
        pick = pick.masked_fill(~kept.repeat_interleave(size, 1), float("-inf"))
    ids = torch.topk(pick, top, dim=-1).indices
    return ids, torch.gather(s, 1, ids)


def route_margin(z: torch.Tensor, correction: torch.Tensor, top: int, groups: Optional[dict]) -> torch.Tensor:
    """[T]: by how much a token's choice is clear: the smallest gap between a pick score that decided for an expert (or a
    group) and the best one that lost; infinite where nothing lost.  A token whose margin is below what rounding moves
    the scores by may go to other experts in an engine that rounds."""
    s = torch.softmax(z, -1)
    pick = s + correction
    T, E = z.shape
    margin = torch.full((T,), float("inf"), dtype=z.dtype)
    if groups:
        size = E // groups["count"]
        best = pick.view(T, groups["count"], size).max(-1).values.sort(-1, descending=True).values
        if groups["keep"] < groups["count"]:
            margin = best[:, groups["keep"] - 1] - best[:, groups["keep"]]
        kept = torch.zeros(T, groups["count"], dtype=torch.bool)
        kept.scatter_(1, torch.topk(pick.view(T, groups["count"], size).max(-1).values, groups["keep"], dim=-1).indices, True)
        pick = pick.masked_fill(~kept.repeat_interleave(size, 1), float("-inf"))
    ordered = pick.sort(-1, descending=True).values
    if top < E:
        gap = ordered[:, top - 1] - ordered[:, top]
        margin = torch.minimum(margin, torch.where(torch.isinf(ordered[:, top]), torch.full_like(gap, float("inf")), gap))
    return margin


def experts(w, pre: str, mlp: dict, x: torch.Tensor, rnd=exact, margins: Optional[list] = None) -> torch.Tensor:
    r = mlp["router"]
    z = x @ w[pre + "router"].T
    ids, weights = route(z, w[pre + "correction"], r["top"], r.get("groups"))
    if margins is not None:
        margins.append(route_margin(z, w[pre + "correction"], r["top"], r.get("groups")))
    y = torch.zeros_like(x)
    for e in range(r["experts"]):
        chosen = (ids == e)
        rows = chosen.any(-1)
        if rows.any():
            share = (weights * chosen).sum(-1)[rows]
            y[rows] += share[:, None] * squared_relu_unit(w, f"{pre}e{e}.", x[rows], rnd)
    if mlp.get("shared"):
        y = y + squared_relu_unit(w, pre + "shared.", x, rnd)
    return y


# ---------------------------------------------------------------------------------------------- the model
def layer_owner(cfg: dict, i: int) -> int:
    """The layer whose tensors layer i uses."""
    while cfg["layers"][i].get("weights_of") is not None:
        i = cfg["layers"][i]["weights_of"]
    return i


def embed(cfg: dict, w, tokens: List[int]) -> torch.Tensor:
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    return tanh_norm(w, "embed.norm", x)


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], coarse: bool = False,
            tap: Optional[list] = None, margins: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``tap`` receives the residual after every layer, ``margins`` every
    router's ``route_margin``."""
    rnd = bf16 if coarse else exact
    eps = cfg["norm"]["eps"]
    x = embed(cfg, w, tokens)
    for i, layer in enumerate(cfg["layers"]):
        name = f"l{layer_owner(cfg, i)}."
        h = rnd(tanh_norm(w, name + "norm1", x))
        if layer["type"] == "attention":
            y = attention(w, name + "mix.", layer["mixer"], eps, h, rnd)
        elif layer["type"] == "attention_2":
            y = attention_2(w, name + "mix.", layer["mixer"], eps, h, rnd)
        else:
            raise ValueError(layer["type"])
        x = x + tanh_norm(w, name + "norm1b", y)
        if layer.get("mlp") is not None:
            h = rnd(tanh_norm(w, name + "norm2", x))
            x = x + tanh_norm(w, name + "norm2b", experts(w, name + "mlp.", layer["mlp"], h, rnd, margins))
        if tap is not None:
            tap.append(x.clone())
    return rnd(tanh_norm(w, "final.norm", x)) @ w["embed"].T * cfg["logit_scale"]
