"""Plain, slow implementation of the Vumalix decoder: whole sequences, no cache, no state carried between calls.

One function per mechanism, float64 throughout, sharing no code with the engine.  ``cfg`` is the parsed
``config.json`` as it stands (nested), ``w`` maps the checkpoint's tensor names to tensors.

Notation: T tokens at positions 0..T-1; H query heads, G key/value heads; dk key size, dv value size per head; a
linear weight W is stored [out, in] and applied as x W^T.

A layer:  x <- x + g1 * unit(mixer(x + conv(x)));  x <- x + g2 * unit(ff(x)), where unit(y) = y / sqrt(mean(y^2) + eps)
and g1, g2 are single numbers.  ``forward(..., coarse=True)`` rounds the activations to bfloat16 where a bfloat16 engine
may: how far that moves a position's logits is the scale of the device tests' bfloat16 tolerance.
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


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def scalar_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    """The layers' and the model's norm: one number for all coordinates."""
    return unit_rms(x, eps) * g.reshape(())


# ---------------------------------------------------------------------------------------------- input convolution
def time_conv(x: torch.Tensor, taps_w: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps_w [C, taps]: y_t = sum_j w[:, j] x_(t - taps + 1 + j), zeros before the first token."""
    T, C = x.shape
    taps = taps_w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += taps_w[:, j] * x[s]
    return y


def mixer_input(x: torch.Tensor, taps_w: Optional[torch.Tensor]) -> torch.Tensor:
    return x if taps_w is None else x + time_conv(x, taps_w)


# ---------------------------------------------------------------------------------------------- rotation
def rotate_half_split(x: torch.Tensor, positions: torch.Tensor, base: float) -> torch.Tensor:
    """x [T, ..., R] with R even: dimension i pairs with i + R/2; the pair (u, v) at position p becomes
    (u cos a - v sin a, v cos a + u sin a), a = p * base^(-2i / R)."""
    R = x.shape[-1]
    half = R // 2
    freq = torch.tensor([base ** (-2.0 * i / R) for i in range(half)], dtype=F64)
    ang = positions.to(F64)[:, None] * freq[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cs, sn = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    u, v = x[..., :half], x[..., half:]
    return torch.cat([u * cs - v * sn, v * cs + u * sn], -1)


def rotate_first(x: torch.Tensor, positions: torch.Tensor, rot: Optional[dict]) -> torch.Tensor:
    """The first rot["dims"] of the last dimension turn, the rest pass unchanged."""
    if not rot or not rot["dims"]:
        return x
    n = rot["dims"]
    return torch.cat([rotate_half_split(x[..., :n], positions, rot["base"]), x[..., n:]], -1)


# ---------------------------------------------------------------------------------------------- softmax attention
def visible(T: int, window: int = 0) -> torch.Tensor:
    """[T, T] truth values: query i sees key j if j <= i and, with a window, i - j < window."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok = ok & (i - j < window)
    return ok


def softmax_heads(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, mask: torch.Tensor) -> torch.Tensor:
    """q [T, H, dk], k [T, H, dk], v [T, H, dv] -> [T, H, dv]."""
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    s = s.masked_fill(~mask[None], float("-inf"))
    p = torch.softmax(s, -1)
    return torch.einsum("hij,jhd->ihd", p, v)


# ---------------------------------------------------------------------------------------------- latent attention
def latent_attention(w, pre: str, m: dict, eps: float, h: torch.Tensor, rnd=exact) -> torch.Tensor:
    """Queries, keys and values through narrow latents; a rotated key part of ``rot_dim`` that all heads share; a
    sliding window; a sigmoid gate on the heads from the mixer's own input."""
    T = h.shape[0]
    H, dk, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = rnd(unit_rms(rnd(h @ w[pre + "dq"].T), eps) * w[pre + "dq.norm"])
    q = rnd(cq @ w[pre + "uq"].T).view(T, H, dk + dr)
    down = rnd(h @ w[pre + "dkv"].T)
    c = rnd(unit_rms(down[:, :rank], eps) * w[pre + "dkv.norm"])
    k_rot = rotate_first(down[:, rank:], pos, m.get("rot"))                  # [T, dr], one for all heads
    q_rot = rotate_first(q[..., dk:], pos, m.get("rot"))
    k_flat = rnd(c @ w[pre + "uk"].T).view(T, H, dk)
    v = rnd(c @ w[pre + "uv"].T).view(T, H, dv)
    qq = rnd(torch.cat([q[..., :dk], q_rot], -1))
    kk = rnd(torch.cat([k_flat, k_rot[:, None, :].expand(T, H, dr)], -1))
    window = (m.get("mask") or {"size": 0})["size"]
    o = softmax_heads(qq, kk, v, m["scale"], visible(T, window)).reshape(T, H * dv)
    gate = torch.sigmoid(rnd(h @ w[pre + "g"].T))
    return rnd(o * gate) @ w[pre + "o"].T


# ---------------------------------------------------------------------------------------------- differential attention
def query_temperature(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * torch.log(torch.floor((positions.to(F64) + 1.0) / every) + 1.0)


def differential_attention(w, pre: str, m: dict, eps: float, h: torch.Tensor, rnd=exact) -> torch.Tensor:
    """Two softmax maps a head over the same values; the second, times lambda, is taken off the first; the difference is
    brought to unit root mean square and scaled by 1 - diff."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(h @ w[pre + "q"].T).view(T, H, 2, dk)
    k = rnd(h @ w[pre + "k"].T).view(T, G, 2, dk)
    v = rnd(h @ w[pre + "v"].T).view(T, G, dv)
    q = unit_rms(q, eps) * w[pre + "q.norm"]
    k = unit_rms(k, eps) * w[pre + "k.norm"]
    temp = m.get("q_temp")
    if temp:
        q = q * query_temperature(torch.arange(T), temp["coef"], temp["every"])[:, None, None, None]
    q, k = rnd(q), rnd(k)
    group = H // G
    kh = k.repeat_interleave(group, 1)      # query head h reads key/value head h // group
    vh = v.repeat_interleave(group, 1)
    mask = visible(T)
    a1 = softmax_heads(q[:, :, 0], kh[:, :, 0], vh, m["scale"], mask)
    a2 = softmax_heads(q[:, :, 1], kh[:, :, 1], vh, m["scale"], mask)
    lam = (torch.exp((w[pre + "lq1"] * w[pre + "lk1"]).sum()) - torch.exp((w[pre + "lq2"] * w[pre + "lk2"]).sum())
           + m["diff"])
    o = unit_rms(a1 - lam * a2, eps) * (1.0 - m["diff"])
    return rnd(o.reshape(T, H * dv)) @ w[pre + "o"].T


# ---------------------------------------------------------------------------------------------- feed-forward
def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N = unit root mean square over the row."""
    a, b, c, e = (coef[i] for i in range(4))
    return a * unit_rms(z, eps) + b * unit_rms(z ** 2, eps) + c * unit_rms(z ** 3, eps) + e


def dense_ff(w, pre: str, eps: float, x: torch.Tensor, rnd=exact) -> torch.Tensor:
    z = rnd(x @ w[pre + "up"].T)
    return rnd(poly_norm(z, w[pre + "act"], eps)) @ w[pre + "down"].T


# ---------------------------------------------------------------------------------------------- the model
def layer_owner(cfg: dict, i: int) -> int:
    """The layer whose tensors layer i uses."""
    while cfg["layers"][i].get("weights_of") is not None:
        i = cfg["layers"][i]["weights_of"]
    return i


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], coarse: bool = False,
            tap: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  ``tap`` receives the residual after every layer."""
    rnd = bf16 if coarse else exact
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)].clone()
    for i, layer in enumerate(cfg["layers"]):
        name = f"l{layer_owner(cfg, i)}."
        h = rnd(mixer_input(x, w.get(name + "canon1")))
        if layer["type"] == "latent_attention":
            y = latent_attention(w, name + "mix.", layer["mixer"], eps, h, rnd)
        elif layer["type"] == "attention":
            y = differential_attention(w, name + "mix.", layer["mixer"], eps, h, rnd)
        else:
            raise ValueError(layer["type"])
        x = x + scalar_norm(y, w[name + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + scalar_norm(dense_ff(w, name + "mlp.", eps, rnd(x), rnd), w[name + "norm2"], eps)
        if tap is not None:
            tap.append(x.clone())
    return rnd(scalar_norm(x, w["final.norm"], eps)) @ w["head"].T
