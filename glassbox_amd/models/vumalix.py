"""The Vumalix decoder assembled from parts.

Every layer norms its sublayers' *outputs* (one number a norm) on their way into the residual (``OutputNormBlock``); the
mixer reads the residual plus a short convolution of it over time (``TimeConv``).  The mixers: attention through narrow
latents with a shared rotated key part and a window (``LatentAttention``), and differential attention
(``DifferentialAttention``); the feed-forward is dense with a polynomial of normed powers (``PolyNormMLP``).  A layer may
use another layer's tensors: the schedule names that layer's block again, with a cache layer (pages and state) of its
own.  Tensor names: ``embed``, ``l<i>.canon1``, ``l<i>.mix.*``, ``l<i>.norm1``, ``l<i>.mlp.*``, ``l<i>.norm2``,
``final.norm``, ``head``, with i the number of the layer that owns them.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.vumalix import VumalixConfig
from ..parts.attention import DifferentialAttention, LatentAttention
from ..parts.block import OutputNormBlock
from ..parts.conv import TimeConv
from ..parts.embedding import Embedding, LMHead
from ..parts.mlp import PolyNormMLP
from ..parts.model import DecoderModel, LayerCall
from ..parts.norm import ScalarRMSNorm


def _mixer(cfg: VumalixConfig, layer):
    m, d, eps = layer["mixer"], cfg.width, cfg.norm_eps
    if layer["type"] == "latent_attention":
        rot = m.get("rot") or {"dims": 0, "base": 1.0}
        return LatentAttention(d, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"], m["scale"],
                               (m.get("mask") or {"size": 0})["size"], rot["dims"], rot["base"], eps)
    temp = m.get("q_temp") or {"coef": 0.0, "every": 0}
    return DifferentialAttention(d, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"], m["diff"], temp["coef"],
                                 temp["every"], eps)


def build_vumalix(cfg: VumalixConfig) -> DecoderModel:
    d, eps = cfg.width, cfg.norm_eps
    owners = [i for i in range(len(cfg.layers)) if cfg.owner(i) == i]   # the layers with tensors of their own, in order
    block_of = {layer: b for b, layer in enumerate(owners)}
    blocks = []
    for i in owners:
        layer = cfg.layers[i]
        ffn = PolyNormMLP(d, layer["mlp"]["ff"], eps) if layer["mlp"] is not None else None
        blocks.append(OutputNormBlock(TimeConv(d, cfg.canon_taps), _mixer(cfg, layer), ScalarRMSNorm(d, eps), ffn,
                                      ScalarRMSNorm(d, eps) if ffn is not None else None))
    schedule = [LayerCall(block=block_of[cfg.owner(i)], cache=i) for i in range(len(cfg.layers))]

    def source(name: str) -> str:
        """The checkpoint numbers a block's tensors by its layer and names a norm or a table by its place alone."""
        if name.endswith(".weight"):
            name = name[:-len(".weight")]
        if name.startswith("blk"):
            b, rest = name[3:].split(".", 1)
            return f"l{owners[int(b)]}.{rest}"
        return name

    return DecoderModel(cfg, Embedding(cfg.vocab, d), blocks, schedule, ScalarRMSNorm(d, eps), LMHead(cfg.vocab, d, any_size=True),
                        names=("embed", "blk{}", "final.norm", "head"), sources=source,
                        arg_keys={"width": "width", "dim": "layers[].mixer.dim", "taps": "canon.taps", "vocab": "vocab"})


register_architecture("Vumalix", VumalixConfig, build_vumalix)
