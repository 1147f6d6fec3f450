"""Small Vumalix configurations for the tests, and how their model folders are made.

Each differs from the others in every option: the convolution of the residual (2 to 5 taps, or none), layers that use
another layer's tensors (one layer three times, two layers in turn, none), latent attention with windows shorter than
a page, across pages and absent, a rotated part of 2 to 32 columns of which all or only some turn, latents narrower and
wider than the heads, heads whose keys are larger or smaller than their values, heads beyond the matrix-core attention;
differential attention with one to four query heads a key head, a temperature that steps every 3, 7 or 40 positions or
is absent, values smaller and larger than two maps; layers without a feed-forward, last and in the middle; a chain of
layers that use another's tensors; sizes that are no multiple of 8.
Score scales are large enough that single keys carry visible weight.
"""
from __future__ import annotations

import os
from typing import Dict

import torch

CASES: Dict[str, dict] = {
    # four taps; layer 0's tensors serve layers 2 and 3; a window across pages; a temperature that steps every 7
    "A": dict(architecture="Vumalix", vocab=211, width=64, norm={"eps": 1e-5}, canon={"taps": 4}, layers=[
        {"type": "latent_attention", "mixer": {"heads": 4, "dim": 24, "rot_dim": 8, "vdim": 16, "q_rank": 24, "kv_rank": 40,
                                               "scale": 0.4, "rot": {"dims": 8, "base": 100.0}, "mask": {"size": 24}},
         "mlp": {"kind": "dense", "ff": 96}},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.5, "diff": 0.3,
                                        "q_temp": {"coef": 0.4, "every": 7}},
         "mlp": {"kind": "dense", "ff": 40}},
        {"type": "latent_attention", "mixer": {"heads": 4, "dim": 24, "rot_dim": 8, "vdim": 16, "q_rank": 24, "kv_rank": 40,
                                               "scale": 0.4, "rot": {"dims": 8, "base": 100.0}, "mask": {"size": 24}},
         "mlp": {"kind": "dense", "ff": 96}, "weights_of": 0},
        {"type": "latent_attention", "mixer": {"heads": 4, "dim": 24, "rot_dim": 8, "vdim": 16, "q_rank": 24, "kv_rank": 40,
                                               "scale": 0.4, "rot": {"dims": 8, "base": 100.0}, "mask": {"size": 24}},
         "mlp": {"kind": "dense", "ff": 96}, "weights_of": 0},
        {"type": "attention", "mixer": {"heads": 3, "kv_heads": 3, "dim": 32, "vdim": 16, "scale": 0.3, "diff": 0.8}, "mlp": None},
    ]),
    # no convolution; every layer its own; no window / a window of 17; only a part of the rotated columns turns; one key head
    # for six query heads; a temperature that steps every 40
    "B": dict(architecture="Vumalix", vocab=130, width=96, norm={"eps": 3e-6}, layers=[
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 1, "dim": 8, "vdim": 48, "scale": 0.6, "diff": 0.5,
                                        "q_temp": {"coef": 1.5, "every": 40}},
         "mlp": {"kind": "dense", "ff": 64}},
        {"type": "latent_attention", "mixer": {"heads": 2, "dim": 16, "rot_dim": 32, "vdim": 64, "q_rank": 48, "kv_rank": 16,
                                               "scale": 0.35, "rot": {"dims": 12, "base": 10000.0}},
         "mlp": None},
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 40, "rot_dim": 8, "vdim": 32, "q_rank": 16, "kv_rank": 64,
                                               "scale": 0.3, "rot": {"dims": 8, "base": 50.0}, "mask": {"size": 17}},
         "mlp": {"kind": "dense", "ff": 32}},
    ]),
    # sizes that the matrix-core products do not take in bfloat16 (inner sizes that are no multiple of 8); two taps; a window
    # shorter than a page; two rotated columns; layers 0 and 1 in turn, twice; a temperature that steps every 3
    "C": dict(architecture="Vumalix", vocab=53, width=50, norm={"eps": 1e-5}, canon={"taps": 2}, layers=[
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 10, "rot_dim": 2, "vdim": 6, "q_rank": 7, "kv_rank": 13,
                                               "scale": 0.9, "rot": {"dims": 2, "base": 20.0}, "mask": {"size": 9}},
         "mlp": {"kind": "dense", "ff": 30}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 6, "vdim": 10, "scale": 0.8, "diff": 0.1,
                                        "q_temp": {"coef": 0.2, "every": 3}},
         "mlp": {"kind": "dense", "ff": 12}},
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 10, "rot_dim": 2, "vdim": 6, "q_rank": 7, "kv_rank": 13,
                                               "scale": 0.9, "rot": {"dims": 2, "base": 20.0}, "mask": {"size": 9}},
         "mlp": {"kind": "dense", "ff": 30}, "weights_of": 0},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 6, "vdim": 10, "scale": 0.8, "diff": 0.1,
                                        "q_temp": {"coef": 0.2, "every": 3}},
         "mlp": {"kind": "dense", "ff": 12}, "weights_of": 1},
    ]),
    # heads of 136 and 144 columns (the plain attention kernel in bfloat16 too); five taps; a window of 50; maps of 72
    "D": dict(architecture="Vumalix", vocab=160, width=128, norm={"eps": 2e-5}, canon={"taps": 5}, layers=[
        {"type": "latent_attention", "mixer": {"heads": 2, "dim": 104, "rot_dim": 32, "vdim": 40, "q_rank": 64, "kv_rank": 32,
                                               "scale": 0.2, "rot": {"dims": 32, "base": 1000.0}, "mask": {"size": 50}},
         "mlp": {"kind": "dense", "ff": 72}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 72, "vdim": 64, "scale": 0.25, "diff": 0.6,
                                        "q_temp": {"coef": 0.3, "every": 16}},
         "mlp": {"kind": "dense", "ff": 256}},
        {"type": "latent_attention", "mixer": {"heads": 8, "dim": 48, "rot_dim": 16, "vdim": 64, "q_rank": 96, "kv_rank": 128,
                                               "scale": 0.25, "rot": {"dims": 16, "base": 10000.0}, "mask": {"size": 33}},
         "mlp": {"kind": "dense", "ff": 64}},
    ]),
    # three taps; layers without a feed-forward in the middle (the mixer's norm is the layer's last pass); a layer that names
    # one which itself uses another's tensors; as many key heads as query heads; no temperature; a window of one page
    "E": dict(architecture="Vumalix", vocab=97, width=72, norm={"eps": 1e-6}, canon={"taps": 3}, layers=[
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 16, "rot_dim": 16, "vdim": 24, "q_rank": 40, "kv_rank": 24,
                                               "scale": 0.3, "rot": {"dims": 16, "base": 500.0}, "mask": {"size": 16}},
         "mlp": None},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 24, "vdim": 40, "scale": 0.4, "diff": 0.7},
         "mlp": {"kind": "dense", "ff": 88}},
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 16, "rot_dim": 16, "vdim": 24, "q_rank": 40, "kv_rank": 24,
                                               "scale": 0.3, "rot": {"dims": 16, "base": 500.0}, "mask": {"size": 16}},
         "mlp": None, "weights_of": 0},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 24, "vdim": 40, "scale": 0.4, "diff": 0.7},
         "mlp": {"kind": "dense", "ff": 88}, "weights_of": 1},
        {"type": "latent_attention", "mixer": {"heads": 3, "dim": 16, "rot_dim": 16, "vdim": 24, "q_rank": 40, "kv_rank": 24,
                                               "scale": 0.3, "rot": {"dims": 16, "base": 500.0}, "mask": {"size": 16}},
         "mlp": None, "weights_of": 2},
    ]),
}


def folder_of(base: str, name: str, seed: int = 0, std: float = 0.05) -> str:
    """Writes (once) the model folder of a case: random matrices, and vectors of sizes that matter (``_spread``)."""
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.weights import write_random_model
    folder = os.path.join(base, f"vumalix_{name}_{seed}")
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        write_random_model(config_from_dict(CASES[name]), folder, seed, std=std, norm_init="uniform", dtype=torch.float32)
        _spread(folder, seed)
    return folder


def _spread(folder: str, seed: int) -> None:
    """The writer draws vectors as small as matrix entries; here they get sizes at which a fault shows: the sublayers'
    norms of the order of the residual (and of either sign), convolution taps of the order of one, the polynomial's four
    numbers all at work, and lambda's vectors large enough that the two exponentials differ."""
    from glassbox_amd.weights import SafetensorsFile, save_file
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    gen = torch.Generator().manual_seed(seed + 1000)
    draw = lambda t, s: torch.randn(t.shape, generator=gen) * s
    for n, t in tensors.items():
        if n.endswith(("norm1", "norm2")):
            tensors[n] = draw(t, 0.1) + 0.15
        elif n.endswith("canon1"):
            tensors[n] = draw(t, 0.6)
        elif n.endswith(".act"):
            tensors[n] = draw(t, 0.5) + torch.tensor([0.6, 0.3, 0.2, 0.1])
        elif n.endswith((".lq1", ".lk1", ".lq2", ".lk2")):
            tensors[n] = draw(t, 0.3)
        elif n == "embed":
            tensors[n] = t * 6.0        # a residual of the order of the sublayers' normed outputs
    save_file(tensors, path)


def rounded(w: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The weights as a bfloat16 engine holds them: matrices rounded, vectors (kept in 32-bit) as they are."""
    return {k: (v.to(torch.bfloat16).to(v.dtype) if v.dim() == 2 and not k.endswith("canon1") else v) for k, v in w.items()}
