"""Configuration of the Vumalix decoder: a list of layers, each with one of two mixers (attention through narrow
latents with a shared rotated key part and a window, or differential attention: two softmax maps a head over the same
values) and a dense feed-forward with a polynomial activation; each sublayer's *output* is normed (one number a norm)
before it joins the residual; the mixer reads the residual plus a short causal convolution of it over time.  A layer
may use another layer's tensors (``weights_of``), with pages and state of its own.

``config.json`` is nested, and this class keeps it as it is read (``layers`` as a tuple of mappings), checked key by
key here so that the builder can rely on it:

  architecture, vocab, width, norm {eps}, canon {taps} (absent: the mixer reads the residual as it is),
  layers[i] {type, mixer {...}, mlp {kind "dense", ff} or null, weights_of (absent: the layer's own tensors)}
    latent_attention: heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot {base, dims}, mask {size} (absent: every
                      earlier key)
    attention:        heads, kv_heads, dim, vdim, scale, diff, q_temp {coef, every} (absent: none)
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig
from .dekinex import _obj
from .sagalorn import _int, _num, _plain

MIXERS = ("latent_attention", "attention")


def _check_layer(i: int, layer: Any) -> Dict[str, Any]:
    where = f"layers[{i}]"
    if not isinstance(layer, dict) or layer.get("type") not in MIXERS or not isinstance(layer.get("mixer"), dict):
        raise ConfigError(f"{where} must have a 'type' out of {', '.join(MIXERS)} and a 'mixer' object")
    kind, m = layer["type"], layer["mixer"]
    mw = f"{where}.mixer"
    out: Dict[str, Any] = {"heads": _int(mw, m, "heads"), "dim": _int(mw, m, "dim")}
    out["vdim"] = _int(mw, m, "vdim", out["dim"])
    if kind == "latent_attention":
        out["rot_dim"] = _int(mw, m, "rot_dim", least=0)
        out["q_rank"], out["kv_rank"] = _int(mw, m, "q_rank"), _int(mw, m, "kv_rank")
        out["scale"] = _num(mw, m, "scale", 1.0 / math.sqrt(out["dim"] + out["rot_dim"]))
        rot = _obj(mw, m, "rot")
        if out["rot_dim"]:
            if rot is None:
                raise ConfigError(f"{mw} has rotated dimensions and lacks the object 'rot'")
            dims = _int(f"{mw}.rot", rot, "dims", out["rot_dim"], least=0)
            if dims % 2 or dims > out["rot_dim"]:
                raise ConfigError(f"{mw}.rot: 'dims' must be even and at most rot_dim, got {dims}")
            out["rot"] = {"dims": dims, "base": _num(f"{mw}.rot", rot, "base")}
            if not out["rot"]["base"] > 0:
                raise ConfigError(f"{mw}.rot: 'base' must be positive")
        mask = _obj(mw, m, "mask")
        if mask is not None:
            out["mask"] = {"size": _int(f"{mw}.mask", mask, "size")}
    else:
        out["kv_heads"] = _int(mw, m, "kv_heads", out["heads"])
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"{mw}: heads ({out['heads']}) is not a multiple of kv_heads ({out['kv_heads']})")
        out["scale"] = _num(mw, m, "scale", 1.0 / math.sqrt(out["dim"]))
        out["diff"] = _num(mw, m, "diff")
        temp = _obj(mw, m, "q_temp")
        if temp is not None:
            out["q_temp"] = {"coef": _num(f"{mw}.q_temp", temp, "coef"), "every": _int(f"{mw}.q_temp", temp, "every")}
    mlp = layer.get("mlp")
    if mlp is not None:
        lw = f"{where}.mlp"
        if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
            raise ConfigError(f"{lw} must be null or an object of kind 'dense', got {mlp!r}")
        mlp = {"kind": "dense", "ff": _int(lw, mlp, "ff")}
    checked = {"type": kind, "mixer": out, "mlp": mlp}
    if layer.get("weights_of") is not None:
        checked["weights_of"] = _int(where, layer, "weights_of", least=0)
    return checked


@dataclass(frozen=True)
class VumalixConfig(ModelConfig):
    architecture = "Vumalix"

    vocab: int
    width: int
    layers: Tuple[Dict[str, Any], ...]
    norm_eps: float
    canon_taps: int = 0

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "VumalixConfig":
        where = "config.json of Vumalix"
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where} lacks a non-empty list 'layers'")
        checked = tuple(_check_layer(i, layer) for i, layer in enumerate(layers))
        for i, layer in enumerate(checked):
            j = layer.get("weights_of")
            if j is None:
                continue
            seen = {i}
            while j is not None and j < len(checked) and j not in seen:   # a layer that itself uses another's: follow it
                seen.add(j)
                last, j = j, checked[j].get("weights_of")
            if j is not None:
                raise ConfigError(f"layers[{i}]: weights_of must lead to another layer with tensors of its own, and leads to layer {j}")
            j = last
            if (checked[j]["type"], checked[j]["mixer"], checked[j]["mlp"]) != (layer["type"], layer["mixer"], layer["mlp"]):
                raise ConfigError(f"layers[{i}] uses the tensors of layer {j} and must equal it in everything else")
        eps = _num("norm", _obj(where, raw, "norm", True), "eps")
        if not eps > 0:
            raise ConfigError("norm: 'eps' must be positive")
        canon = _obj(where, raw, "canon")
        taps = _int("canon", canon, "taps") if canon is not None else 0
        return cls(vocab=_int(where, raw, "vocab"), width=_int(where, raw, "width"), layers=checked, norm_eps=eps,
                   canon_taps=taps)

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            entry = {"type": l["type"], "mixer": _plain(l["mixer"]), "mlp": _plain(l["mlp"])}
            if l.get("weights_of") is not None:
                entry["weights_of"] = l["weights_of"]
            layers.append(entry)
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.canon_taps:
            out["canon"] = {"taps": self.canon_taps}
        return out

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i uses."""
        while self.layers[i].get("weights_of") is not None:
            i = self.layers[i]["weights_of"]
        return i
