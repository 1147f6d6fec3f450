"""The Tekilix decoder assembled from parts.

Every sublayer stands between two bounded norms (``SandwichBlock`` of ``TanhNorm``s): x += n1b(mixer(n1(x))), then
x += n2b(experts(n2(x))).  Both mixers are ``GatedAttention`` with other options: *attention* has biased projections, one
RMS norm over all of q (and of k), neighbouring pairs that turn, capped scores, a sink of score 0 and one gate a head;
*attention_2* passes q and k through a short convolution over time, takes the convolved keys as values, norms head by
head, turns halves of the rotated channels with stretched slow frequencies, has a learned sink a head and a gate a
channel.  Both see the keys of their own run of ``mask.size`` positions.  The feed-forward is ``RoutedExperts`` with
softmax scores, a choice among the best groups of experts, weights that are the scores as they stand, squared-ReLU
units and a shared expert that always counts.  The embedding is scaled and normed, and its table is the head, whose
logits are scaled.  A layer may use another layer's tensors: the schedule names that layer's block again, with a cache
layer (pages and state) of its own.  Tensor names: ``embed``, ``embed.norm[.b|.alpha]``, ``l<i>.norm1`` (``norm1b``,
``norm2``, ``norm2b``), ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, with i the number of the layer that owns them.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.tekilix import TekilixConfig
from ..parts.attention import GatedAttention
from ..parts.block import SandwichBlock
from ..parts.embedding import Embedding, LMHead
from ..parts.model import DecoderModel, LayerCall
from ..parts.moe import RoutedExperts
from ..parts.norm import TanhNorm


def _mixer(cfg: TekilixConfig, layer) -> GatedAttention:
    m, d, eps = layer["mixer"], cfg.width, cfg.norm_eps
    rot = m.get("rot") or {"dims": 0, "base": 10000.0}
    chunk = (m.get("mask") or {"size": 0})["size"]
    common = dict(rot_dims=rot["dims"], rot_base=rot["base"], chunk=chunk)
    if layer["type"] == "attention":
        return GatedAttention(d, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], eps, bias=True, qk_norm="joint",
                              rot_pairs="neighbours", softcap=m.get("softcap", 0.0), sink="zero", gate="head", **common)
    sc = rot.get("scaling")
    scaling = (sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else None
    return GatedAttention(d, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], eps, taps=m.get("conv", 0),
                          tied_values=True, qk_norm="head", rot_pairs="halves", rot_scaling=scaling, sink="learned",
                          gate="channel", **common)


def _experts(cfg: TekilixConfig, mlp) -> RoutedExperts:
    r = mlp["router"]
    groups = (r["groups"]["count"], r["groups"]["keep"]) if r.get("groups") else None
    return RoutedExperts(cfg.width, r["experts"], r["top"], mlp["expert"]["ff"], 1.0, (mlp.get("shared") or {"ff": 0})["ff"],
                         correction=True, scoring="softmax", renorm=False, groups=groups, unit="relu2", shared_gate=False)


def build_tekilix(cfg: TekilixConfig) -> DecoderModel:
    d = cfg.width
    owners = [i for i in range(len(cfg.layers)) if cfg.owner(i) == i]   # the layers with tensors of their own, in order
    block_of = {layer: b for b, layer in enumerate(owners)}
    blocks = []
    for i in owners:
        layer = cfg.layers[i]
        ffn = _experts(cfg, layer["mlp"]) if layer["mlp"] is not None else None
        blocks.append(SandwichBlock(TanhNorm(d), _mixer(cfg, layer), TanhNorm(d), TanhNorm(d) if ffn is not None else None, ffn,
                                    TanhNorm(d) if ffn is not None else None))
    schedule = [LayerCall(block=block_of[cfg.owner(i)], cache=i) for i in range(len(cfg.layers))]

    def source(name: str) -> str:
        """The checkpoint numbers a block's tensors by its layer, names a norm's weight by the norm alone and its bias
        ``.b``."""
        if name.startswith("blk"):
            b, rest = name[3:].split(".", 1)
            name = f"l{owners[int(b)]}.{rest}"
        if name.endswith(".weight"):
            return name[:-len(".weight")]
        if name.endswith(".bias"):
            return name[:-len(".bias")] + ".b"
        return name

    embedding = Embedding(cfg.vocab, d, scale=cfg.embedding_scale, norm=TanhNorm(d))
    return DecoderModel(cfg, embedding, blocks, schedule, TanhNorm(d),
                        LMHead(cfg.vocab, d, tied_to=embedding, scale=cfg.logit_scale, any_size=True),
                        names=("embed", "blk{}", "final.norm", "head"), sources=source,
                        arg_keys={"width": "width", "dim": "layers[].mixer.dim", "taps": "layers[].mixer.conv", "vocab": "vocab",
                                  "n_experts": "layers[].mlp.router.experts", "top": "layers[].mlp.router.top"})


register_architecture("Tekilix", TekilixConfig, build_tekilix)
