"""Configuration of the Tekilix decoder: a list of layers, each with one of two gated attention mixers and an optional
feed-forward of routed experts; bounded norms (tanh(alpha x) * w + b) before and after every sublayer, behind the
embedding and before the head; a scaled embedding whose table is also the head, with scaled logits.  A layer may use
another layer's tensors (``weights_of``), with pages and state of its own.

``config.json`` is nested, and this class keeps it as it is read (``layers`` as a tuple of mappings), checked key by
key here so that the builder can rely on it:

  architecture, vocab, width, norm {eps}, embedding {scale}, logit_scale,
  layers[i] {type, mixer {...}, mlp {...} or null, weights_of (absent: the layer's own tensors)}
    attention:    heads, kv_heads, dim, vdim, scale, softcap (absent: none), rot {base, dims} (absent: none),
                  mask {size} (absent: every earlier key)
    attention_2:  heads, kv_heads, dim, vdim (= dim: the values are the keys), scale, conv (taps; absent: none),
                  rot {base, dims, scaling {factor, original, fast, slow} (absent: none)}, mask {size}
    mlp:          kind "moe", expert {ff}, router {experts, top, groups {count, keep} (absent: none)},
                  shared {ff} (absent: none)
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Tuple

from .base import ConfigError, ModelConfig
from .dekinex import _obj
from .sagalorn import _int, _num, _plain

MIXERS = ("attention", "attention_2")


def _check_rot(mw: str, m: Dict[str, Any], dim: int, scaling_allowed: bool):
    rot = _obj(mw, m, "rot")
    if rot is None:
        return None
    where = f"{mw}.rot"
    dims = _int(where, rot, "dims", least=0)
    if dims % 2 or dims > dim:
        raise ConfigError(f"{where}: 'dims' must be even and at most dim ({dim}), got {dims}")
    if dims == 0:
        return None
    out = {"dims": dims, "base": _num(where, rot, "base")}
    if not out["base"] > 1:
        raise ConfigError(f"{where}: 'base' must be above 1")
    sc = _obj(where, rot, "scaling")
    if sc is not None:
        if not scaling_allowed:
            raise ConfigError(f"{where}: 'scaling' goes with the mixer attention_2")
        out["scaling"] = {k: _num(f"{where}.scaling", sc, k) for k in ("factor", "original", "fast", "slow")}
        if any(not v > 0 for v in out["scaling"].values()):
            raise ConfigError(f"{where}.scaling: factor, original, fast and slow must be positive")
    return out


def _check_mlp(where: str, mlp: Any):
    if mlp is None:
        return None
    if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
        raise ConfigError(f"{where} must be null or an object of kind 'moe', got {mlp!r}")
    router = _obj(where, mlp, "router", True)
    rw = f"{where}.router"
    out = {"kind": "moe", "expert": {"ff": _int(f"{where}.expert", _obj(where, mlp, "expert", True), "ff")},
           "router": {"experts": _int(rw, router, "experts"), "top": _int(rw, router, "top")}}
    E, top = out["router"]["experts"], out["router"]["top"]
    if top > E:
        raise ConfigError(f"{rw}: 'top' ({top}) is above 'experts' ({E})")
    groups = _obj(rw, router, "groups")
    if groups is not None:
        count, keep = _int(f"{rw}.groups", groups, "count"), _int(f"{rw}.groups", groups, "keep")
        if E % count or keep > count or keep * (E // count) < top:
            raise ConfigError(f"{rw}.groups: {E} experts in {count} groups of which {keep} are kept cannot give {top} a token")
        out["router"]["groups"] = {"count": count, "keep": keep}
    shared = _obj(where, mlp, "shared")
    if shared is not None:
        out["shared"] = {"ff": _int(f"{where}.shared", shared, "ff")}
    return out


def _check_layer(i: int, layer: Any) -> Dict[str, Any]:
    where = f"layers[{i}]"
    if not isinstance(layer, dict) or layer.get("type") not in MIXERS or not isinstance(layer.get("mixer"), dict):
        raise ConfigError(f"{where} must have a 'type' out of {', '.join(MIXERS)} and a 'mixer' object")
    kind, m = layer["type"], layer["mixer"]
    mw = f"{where}.mixer"
    out: Dict[str, Any] = {"heads": _int(mw, m, "heads"), "dim": _int(mw, m, "dim")}
    out["kv_heads"] = _int(mw, m, "kv_heads", out["heads"])
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{mw}: heads ({out['heads']}) is not a multiple of kv_heads ({out['kv_heads']})")
    out["vdim"] = _int(mw, m, "vdim", out["dim"])
    out["scale"] = _num(mw, m, "scale", 1.0 / math.sqrt(out["dim"]))
    rot = _check_rot(mw, m, out["dim"], kind == "attention_2")
    if rot is not None:
        out["rot"] = rot
    mask = _obj(mw, m, "mask")
    if mask is not None:
        out["mask"] = {"size": _int(f"{mw}.mask", mask, "size")}
    if kind == "attention":
        if m.get("softcap") is not None:
            out["softcap"] = _num(mw, m, "softcap")
            if not out["softcap"] > 0:
                raise ConfigError(f"{mw}: 'softcap' must be positive")
    else:
        if out["vdim"] != out["dim"]:
            raise ConfigError(f"{mw}: the values of attention_2 are its keys, so 'vdim' ({out['vdim']}) must equal 'dim' ({out['dim']})")
        if m.get("conv") is not None:
            out["conv"] = _int(mw, m, "conv")
    checked = {"type": kind, "mixer": out, "mlp": _check_mlp(f"{where}.mlp", layer.get("mlp"))}
    if layer.get("weights_of") is not None:
        checked["weights_of"] = _int(where, layer, "weights_of", least=0)
    return checked


@dataclass(frozen=True)
class TekilixConfig(ModelConfig):
    architecture = "Tekilix"

    vocab: int
    width: int
    layers: Tuple[Dict[str, Any], ...]
    norm_eps: float
    embedding_scale: float = 1.0
    logit_scale: float = 1.0

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "TekilixConfig":
        where = "config.json of Tekilix"
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where} lacks a non-empty list 'layers'")
        checked = tuple(_check_layer(i, layer) for i, layer in enumerate(layers))
        for i, layer in enumerate(checked):
            j = layer.get("weights_of")
            if j is None:
                continue
            seen, last = {i}, i
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
        emb = _obj(where, raw, "embedding")
        return cls(vocab=_int(where, raw, "vocab"), width=_int(where, raw, "width"), layers=checked, norm_eps=eps,
                   embedding_scale=_num("embedding", emb, "scale", 1.0) if emb is not None else 1.0,
                   logit_scale=_num(where, raw, "logit_scale", 1.0))

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            entry = {"type": l["type"], "mixer": _plain(l["mixer"]), "mlp": _plain(l["mlp"])}
            if l.get("weights_of") is not None:
                entry["weights_of"] = l["weights_of"]
            layers.append(entry)
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale, "layers": layers}

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i uses."""
        while self.layers[i].get("weights_of") is not None:
            i = self.layers[i]["weights_of"]
        return i
