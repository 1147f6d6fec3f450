"""Small Tekilix configurations for the tests, and how their model folders are made.

Each differs from the others in every option: the two mixers in any order and number; one to six query heads a key
head; key sizes above and below value sizes, heads that are no multiple of 16 and heads beyond the matrix-core
attention; rotation of a part of the head, of all of it, of two channels, or none; stretched frequencies or plain
ones; runs of positions shorter than a page, a page long, across pages, and no runs at all; capped scores or not; one to
five taps, or no convolution; three to sixteen experts, one to all of them a token, groups of one to four experts of
which some or all are kept, or no groups; a shared expert or none; layers without a feed-forward, last and in the
middle; layers that use another layer's tensors, also through a chain; sizes that are no multiple of 8; embedding and
logit scales on both sides of 1.
Score scales are large enough that single keys carry visible weight.
"""
from __future__ import annotations

import os
from typing import Dict

import torch


def _moe(experts, top, ff, groups=None, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if groups:
        out["router"]["groups"] = {"count": groups[0], "keep": groups[1]}
    if shared:
        out["shared"] = {"ff": shared}
    return out


_A0 = {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 24, "vdim": 16, "scale": 0.4, "softcap": 4.0,
                                      "rot": {"dims": 8, "base": 100.0}, "mask": {"size": 24}},
       "mlp": _moe(6, 2, 24, (3, 2), 40)}
_A1 = {"type": "attention_2", "mixer": {"heads": 4, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.5, "conv": 4,
                                        "rot": {"dims": 16, "base": 1000.0,
                                                "scaling": {"factor": 8.0, "original": 64, "fast": 4.0, "slow": 1.0}},
                                        "mask": {"size": 50}},
       "mlp": _moe(4, 4, 16)}
_C0 = {"type": "attention_2", "mixer": {"heads": 3, "kv_heads": 3, "dim": 10, "vdim": 10, "scale": 0.9, "conv": 2,
                                        "rot": {"dims": 2, "base": 20.0}, "mask": {"size": 9}},
       "mlp": _moe(3, 1, 30)}
_C1 = {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 6, "vdim": 10, "scale": 0.8,
                                      "rot": {"dims": 6, "base": 50.0}, "mask": {"size": 7}},
       "mlp": _moe(5, 3, 12, None, 20)}
_E0 = {"type": "attention", "mixer": {"heads": 3, "kv_heads": 3, "dim": 16, "vdim": 48, "scale": 0.3, "softcap": 1.5,
                                      "rot": {"dims": 16, "base": 500.0}, "mask": {"size": 16}},
       "mlp": None}
_E1 = {"type": "attention_2", "mixer": {"heads": 2, "kv_heads": 2, "dim": 24, "vdim": 24, "scale": 0.4, "conv": 3,
                                        "rot": {"dims": 12, "base": 300.0,
                                                "scaling": {"factor": 2.0, "original": 32, "fast": 8.0, "slow": 2.0}},
                                        "mask": {"size": 40}},
       "mlp": _moe(8, 3, 24, (2, 1), 16)}

CASES: Dict[str, dict] = {
    # both mixers in turn, each used twice; runs of 24 and 50 positions; part of the head and all of it rotated; groups of
    # two experts; a router that takes all four experts; a last layer without a feed-forward
    "A": dict(architecture="Tekilix", vocab=211, width=64, norm={"eps": 1e-5}, embedding={"scale": 3.0}, logit_scale=0.5,
              layers=[_A0, _A1, dict(_A0, weights_of=0), dict(_A1, weights_of=1),
                      {"type": "attention", "mixer": {"heads": 3, "kv_heads": 3, "dim": 32, "vdim": 32, "scale": 0.3, "softcap": 50.0,
                                                      "mask": {"size": 100}},
                       "mlp": None}]),
    # no runs of positions (every earlier key) in one layer, no cap, no convolution, no stretching; one key head for six
    # query heads; as many key heads as query heads; one group (nothing to leave out) and groups that are all kept
    "B": dict(architecture="Tekilix", vocab=130, width=96, norm={"eps": 3e-6}, embedding={"scale": 0.7}, logit_scale=2.0,
              layers=[
                  {"type": "attention", "mixer": {"heads": 6, "kv_heads": 1, "dim": 8, "vdim": 48, "scale": 0.6,
                                                  "rot": {"dims": 4, "base": 10000.0}},
                   "mlp": _moe(4, 2, 64, (1, 1))},
                  {"type": "attention_2", "mixer": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.2,
                                                    "rot": {"dims": 32, "base": 10000.0}, "mask": {"size": 33}},
                   "mlp": None},
                  {"type": "attention_2", "mixer": {"heads": 3, "kv_heads": 1, "dim": 40, "vdim": 40, "scale": 0.3, "conv": 1,
                                                    "mask": {"size": 17}},
                   "mlp": _moe(12, 5, 16, (4, 4), 32)},
              ]),
    # sizes that the matrix-core products do not take in bfloat16 (inner sizes that are no multiple of 8); runs shorter
    # than a page; two rotated channels and a whole head of six; two layers in turn, twice; one expert a token
    "C": dict(architecture="Tekilix", vocab=53, width=50, norm={"eps": 1e-5}, embedding={"scale": 1.0}, logit_scale=1.0,
              layers=[_C0, _C1, dict(_C0, weights_of=0), dict(_C1, weights_of=1)]),
    # heads of 136 and 144 channels (the plain attention kernel in bfloat16 too); five taps; sixteen experts in four
    # groups of which two are kept; eight query heads a key head
    "D": dict(architecture="Tekilix", vocab=160, width=128, norm={"eps": 2e-5}, embedding={"scale": 12.0}, logit_scale=0.1,
              layers=[
                  {"type": "attention_2", "mixer": {"heads": 2, "kv_heads": 1, "dim": 136, "vdim": 136, "scale": 0.2, "conv": 5,
                                                    "rot": {"dims": 32, "base": 1000.0,
                                                            "scaling": {"factor": 16.0, "original": 128, "fast": 16.0, "slow": 1.0}},
                                                    "mask": {"size": 64}},
                   "mlp": _moe(16, 3, 8, (4, 2), 72)},
                  {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 144, "vdim": 64, "scale": 0.15, "softcap": 8.0,
                                                  "rot": {"dims": 64, "base": 10000.0}, "mask": {"size": 33}},
                   "mlp": _moe(4, 1, 256)},
                  {"type": "attention", "mixer": {"heads": 8, "kv_heads": 1, "dim": 48, "vdim": 64, "scale": 0.25, "softcap": 2.0,
                                                  "rot": {"dims": 16, "base": 10000.0}, "mask": {"size": 200}},
                   "mlp": _moe(8, 8, 16, (8, 8))},
              ]),
    # layers without a feed-forward in the middle; a layer that names one which itself uses another's tensors; values
    # larger than keys; runs of one page; one group of two kept
    "E": dict(architecture="Tekilix", vocab=97, width=72, norm={"eps": 1e-6}, embedding={"scale": 5.0}, logit_scale=0.25,
              layers=[_E0, _E1, dict(_E0, weights_of=0), dict(_E1, weights_of=1), dict(_E0, weights_of=2)]),
}


def folder_of(base: str, name: str, seed: int = 0, std: float = 0.05) -> str:
    """Writes (once) the model folder of a case: random matrices, and vectors of sizes that matter (``_spread``)."""
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.weights import write_random_model
    folder = os.path.join(base, f"tekilix_{name}_{seed}")
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        write_random_model(config_from_dict(CASES[name]), folder, seed, std=std, norm_init="uniform", dtype=torch.float32)
        _spread(folder, seed)
    return folder


def _spread(folder: str, seed: int) -> None:
    """The writer draws vectors as small as matrix entries; here they get sizes at which a fault shows: norm biases and
    the projections' biases of the order of what they are added to, norm weights of either sign, convolution taps of
    the order of one, sinks that take a visible share, corrections that change which experts are chosen, and
    projections large enough that scores spread out."""
    from glassbox_amd.weights import SafetensorsFile, save_file
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    gen = torch.Generator().manual_seed(seed + 1000)
    draw = lambda t, s: torch.randn(t.shape, generator=gen) * s
    for n, t in tensors.items():
        last = n.rsplit(".", 1)[-1]
        if n.endswith((".norm1b", ".norm2b")):
            tensors[n] = draw(t, 0.3) + 0.4
        elif n.endswith(("norm1.b", "norm2.b", "embed.norm.b")):
            tensors[n] = draw(t, 0.1)
        elif n.endswith(("norm1b.b", "norm2b.b", "final.norm.b")):
            tensors[n] = draw(t, 0.03)    # (the same for every token: larger, and every reply is the same token)
        elif n.endswith((".q.b", ".k.b")):
            tensors[n] = draw(t, 0.5)
        elif n.endswith(".v.b"):
            tensors[n] = draw(t, 0.1)
        elif n.endswith(".conv"):
            tensors[n] = draw(t, 0.6)
        elif last == "sink":
            tensors[n] = draw(t, 1.0)
        elif last == "correction":
            tensors[n] = draw(t, 0.05)
        elif last in ("q", "k", "router", "g") and ".mix." in n or last == "router":
            tensors[n] = t * 6.0
        elif last in ("up", "down", "v", "o"):
            tensors[n] = t * 3.0
    save_file(tensors, path)


def rounded(w: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The weights as a bfloat16 engine holds them: matrices rounded, vectors and the convolutions' taps (kept in 32-bit)
    as they are."""
    return {k: (v.to(torch.bfloat16).to(v.dtype) if v.dim() == 2 and not k.endswith(".conv") else v) for k, v in w.items()}
