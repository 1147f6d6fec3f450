"""Vumalix without a device: the plain implementation pinned by what fixes it beside its own text, the configuration's
checks, the tensors the model declares, and the order of its layer calls."""
from __future__ import annotations

import copy
import math

import pytest
import torch

from plain import vumalix as pv
from vumalix_cases import CASES, folder_of

F64 = torch.float64


# ------------------------------------------------------------------------------------------ the plain implementation
def test_the_convolution_over_time_is_a_causal_correlation():
    torch.manual_seed(0)
    x, taps = torch.randn(11, 5, dtype=F64), torch.randn(5, 4, dtype=F64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.t()[None], (3, 0)), taps[:, None, :], groups=5)[0].t()
    assert torch.allclose(pv.time_conv(x, taps), want, atol=1e-12)
    # the last tap weighs the token itself, the first the oldest; the mixer reads the residual plus that
    one = torch.zeros(6, 1, dtype=F64)
    one[2] = 1.0
    w = torch.tensor([[1.0, 10.0, 100.0]], dtype=F64)
    assert pv.time_conv(one, w)[:, 0].tolist() == [0.0, 0.0, 100.0, 10.0, 1.0, 0.0]
    assert pv.mixer_input(one, w)[:, 0].tolist() == [0.0, 0.0, 101.0, 10.0, 1.0, 0.0]
    assert torch.equal(pv.mixer_input(one, None), one)


def test_rotation_pairs_the_halves_and_scores_depend_on_the_distance_alone():
    x = torch.zeros(3, 1, 6, dtype=F64)
    x[:, 0, 0] = 1.0                       # (1, 0) in the pair (0, 3)
    out = pv.rotate_half_split(x, torch.arange(3), 100.0)
    for t in range(3):
        assert out[t, 0, 0] == pytest.approx(math.cos(t)) and out[t, 0, 3] == pytest.approx(math.sin(t))
        assert out[t, 0, 1] == 0.0 and out[t, 0, 4] == 0.0
    y = torch.zeros(2, 4, dtype=F64)
    y[:, 1] = 1.0                          # the second pair turns at base^(-2/4) a position
    got = pv.rotate_half_split(y, torch.tensor([0, 5]), 16.0)
    assert got[1, 1] == pytest.approx(math.cos(5 / 4.0)) and got[1, 3] == pytest.approx(math.sin(5 / 4.0))
    torch.manual_seed(1)
    q, k = torch.randn(1, 2, 8, dtype=F64).expand(9, 2, 8), torch.randn(1, 2, 8, dtype=F64).expand(9, 2, 8)
    rq, rk = pv.rotate_half_split(q, torch.arange(9), 50.0), pv.rotate_half_split(k, torch.arange(9), 50.0)
    assert torch.allclose((rq[5] * rk[2]).sum(-1), (rq[8] * rk[5]).sum(-1), atol=1e-12)
    assert not torch.allclose((rq[5] * rk[2]).sum(-1), (rq[5] * rk[4]).sum(-1), atol=1e-3)


def test_visibility_at_the_windows_edges():
    see = pv.visible(12, 4)
    assert see[10, 10] and see[10, 7] and not see[10, 6] and not see[10, 11]
    assert pv.visible(12)[11, 0] and not pv.visible(12)[3, 4]
    one = pv.visible(6, 1)
    assert one[5, 5] and not one[5, 4]


def test_softmax_attention_is_the_library_routine():
    torch.manual_seed(2)
    T, H, dk, dv = 9, 3, 5, 4
    q, k, v = torch.randn(T, H, dk, dtype=F64), torch.randn(T, H, dk, dtype=F64), torch.randn(T, H, dv, dtype=F64)
    for window in (0, 3):
        mask = pv.visible(T, window)
        want = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                                                attn_mask=mask, scale=0.7).transpose(0, 1)
        assert torch.allclose(pv.softmax_heads(q, k, v, 0.7, mask), want, atol=1e-12)


def test_the_temperature_steps_with_the_position():
    t = pv.query_temperature(torch.arange(20), 0.5, 7)
    assert t[0] == 1.0 and t[5] == 1.0                        # floor(6 / 7) = 0
    assert t[6] == pytest.approx(1 + 0.5 * math.log(2))       # position 6 is the seventh token
    assert t[13] == pytest.approx(1 + 0.5 * math.log(3)) and t[12] == t[6]


def test_the_polynomial_of_normed_powers():
    torch.manual_seed(3)
    z = torch.randn(4, 10, dtype=F64)
    unit = lambda v: v / torch.sqrt((v * v).mean(-1, keepdim=True) + 1e-5)
    assert torch.allclose(pv.poly_norm(z, torch.tensor([1.0, 0, 0, 0], dtype=F64), 1e-5), unit(z))
    assert torch.allclose(pv.poly_norm(z, torch.tensor([0, 1.0, 0, 0], dtype=F64), 1e-5), unit(z * z))
    assert torch.allclose(pv.poly_norm(z, torch.tensor([0, 0, 2.0, 0.25], dtype=F64), 1e-5), 2 * unit(z ** 3) + 0.25)


def test_latent_attention_with_one_token_and_with_wide_latents():
    """A single token attends to itself alone: the mixer is then the gate times the value path, whatever queries and keys
    are.  And with nothing rotated and orthogonal up-projections the scores are those of the latents themselves."""
    torch.manual_seed(4)
    d, H, dk, dr, dv, rq, rk = 12, 2, 4, 2, 3, 5, 6
    m = {"heads": H, "dim": dk, "rot_dim": dr, "vdim": dv, "q_rank": rq, "kv_rank": rk, "scale": 0.5, "rot": {"dims": dr, "base": 10.0}}
    w = {"dq": torch.randn(rq, d), "dq.norm": torch.rand(rq) + 0.5, "uq": torch.randn(H * (dk + dr), rq), "dkv": torch.randn(rk + dr, d),
         "dkv.norm": torch.rand(rk) + 0.5, "uk": torch.randn(H * dk, rk), "uv": torch.randn(H * dv, rk), "g": torch.randn(H * dv, d),
         "o": torch.randn(d, H * dv)}
    w = {k: v.to(F64) for k, v in w.items()}
    h = torch.randn(1, d, dtype=F64)
    c = pv.unit_rms(h @ w["dkv"].T[:, :rk], 1e-6) * w["dkv.norm"]
    want = ((c @ w["uv"].T) * torch.sigmoid(h @ w["g"].T)) @ w["o"].T
    assert torch.allclose(pv.latent_attention(w, "", m, 1e-6, h), want, atol=1e-12)
    # the shared rotated part reaches every head: doubling it changes the outputs of a longer sequence
    hs = torch.randn(7, d, dtype=F64)
    w2 = dict(w)
    w2["dkv"] = w["dkv"].clone()
    w2["dkv"][rk:] *= 2.0
    assert not torch.allclose(pv.latent_attention(w2, "", m, 1e-6, hs), pv.latent_attention(w, "", m, 1e-6, hs), atol=1e-6)
    # a window of one leaves every token its own value path
    m1 = dict(m, mask={"size": 1})
    c = pv.unit_rms(hs @ w["dkv"].T[:, :rk], 1e-6) * w["dkv.norm"]
    assert torch.allclose(pv.latent_attention(w, "", m1, 1e-6, hs), ((c @ w["uv"].T) * torch.sigmoid(hs @ w["g"].T)) @ w["o"].T, atol=1e-12)


def test_differential_attention_takes_the_second_map_off_the_first():
    torch.manual_seed(5)
    d, H, G, dk, dv, T = 10, 4, 2, 3, 5, 8
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 0.8, "diff": 0.25}
    w = {"q": torch.randn(H * 2 * dk, d), "k": torch.randn(G * 2 * dk, d), "v": torch.randn(G * dv, d), "o": torch.randn(d, H * dv),
         "q.norm": torch.rand(dk) + 0.5, "k.norm": torch.rand(dk) + 0.5, "lq1": torch.randn(dk) * 0.4, "lk1": torch.randn(dk) * 0.4,
         "lq2": torch.randn(dk) * 0.4, "lk2": torch.randn(dk) * 0.4}
    w = {k: v.to(F64) for k, v in w.items()}
    h = torch.randn(T, d, dtype=F64)
    got = pv.differential_attention(w, "", m, 1e-6, h)
    # written out head by head with the library's attention
    q = (h @ w["q"].T).view(T, H, 2, dk)
    k = (h @ w["k"].T).view(T, G, 2, dk)
    v = (h @ w["v"].T).view(T, G, dv)
    lam = math.exp(float(w["lq1"] @ w["lk1"])) - math.exp(float(w["lq2"] @ w["lk2"])) + 0.25
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        maps = []
        for mp in range(2):
            qq = pv.unit_rms(q[:, hh, mp], 1e-6) * w["q.norm"]
            kk = pv.unit_rms(k[:, g, mp], 1e-6) * w["k.norm"]
            maps.append(torch.nn.functional.scaled_dot_product_attention(qq[None], kk[None], v[None, :, g], is_causal=True, scale=0.8)[0])
        o = maps[0] - lam * maps[1]
        heads.append(o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6) * 0.75)
    assert torch.allclose(got, torch.cat(heads, -1) @ w["o"].T, atol=1e-10)
    # equal maps and lambda 1 would cancel: with lq, lk zero lambda is diff alone
    w0 = dict(w, lq1=torch.zeros(dk, dtype=F64), lq2=torch.zeros(dk, dtype=F64))
    m0 = dict(m, diff=0.0)
    only_first = pv.differential_attention(w0, "", m0, 1e-6, h)
    w0["k"] = w["k"].clone()
    w0["k"].view(G, 2, dk, d)[:, 1] = 0.0   # the second map's keys do not matter when lambda is zero
    assert torch.allclose(pv.differential_attention(w0, "", m0, 1e-6, h), only_first, atol=1e-12)


@pytest.mark.parametrize("name", list(CASES))
def test_the_plain_model_is_causal_and_its_parts_all_matter(model_dirs, name):
    """A later token changes no earlier logits; every tensor of the checkpoint changes the last logits when it is
    disturbed (a part that the forward pass forgot would not)."""
    folder = folder_of(model_dirs.base, name)
    cfg, w = pv.load_folder(folder)
    toks = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7, 9, 3, 2, 3, 8, 4, 6, 2, 6, 4, 3, 3, 8, 3, 2, 7, 9, 5, 0, 2, 8, 8, 4, 1, 9, 7]
    toks = [t % cfg["vocab"] for t in toks]
    base = pv.forward(cfg, w, toks)
    other = pv.forward(cfg, w, toks[:-1] + [(toks[-1] + 1) % cfg["vocab"]])
    assert torch.equal(base[:-1], other[:-1]) and not torch.equal(base[-1], other[-1])
    assert torch.allclose(base[:17], pv.forward(cfg, w, toks[:17]), atol=1e-12)
    for n in sorted(w):
        if n in ("embed", "head"):
            continue   # (tables: most rows are not read by forty tokens)
        w2 = dict(w)
        w2[n] = w[n] + 0.9 * torch.cos(1.7 * torch.arange(w[n].numel(), dtype=F64) + 0.3).view_as(w[n])
        assert not torch.allclose(pv.forward(cfg, w2, toks)[-1], base[-1], atol=1e-9), n
    # the residual after every layer call, and a layer that uses another's tensors is a call of its own
    tap = []
    pv.forward(cfg, w, toks, tap=tap)
    assert len(tap) == len(cfg["layers"]) and all(not torch.equal(a, b) for a, b in zip(tap, tap[1:]))


# ------------------------------------------------------------------------------------------ configuration and tensors
def test_the_configuration_is_checked_key_by_key():
    from glassbox_amd.config import ConfigError, config_from_dict
    cfg = config_from_dict(CASES["A"])
    assert cfg.architecture == "Vumalix" and cfg.canon_taps == 4 and [cfg.owner(i) for i in range(5)] == [0, 1, 0, 0, 4]
    assert config_from_dict(cfg.to_dict()) == cfg
    assert config_from_dict(CASES["B"]).canon_taps == 0
    assert [config_from_dict(CASES["C"]).owner(i) for i in range(4)] == [0, 1, 0, 1]

    def broken(path, value):
        raw = copy.deepcopy(CASES["A"])
        at = raw
        for key in path[:-1]:
            at = at[key]
        if value is None:
            at.pop(path[-1])
        else:
            at[path[-1]] = value
        return raw
    # a layer may name one that itself uses another's tensors: the chain is followed to the layer that owns them
    assert [config_from_dict(broken(("layers", 3, "weights_of"), 2)).owner(i) for i in range(5)] == [0, 1, 0, 0, 4]
    for path, value, word in ((("layers", 0, "type"), "conv", "type"), (("layers", 1, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 0, "mixer", "rot", "dims"), 7, "dims"), (("layers", 0, "mixer", "kv_rank"), None, "kv_rank"),
                              (("layers", 1, "mixer", "diff"), None, "diff"), (("layers", 1, "mixer", "q_temp", "every"), 0, "every"),
                              (("layers", 3, "weights_of"), 3, "weights_of"), (("layers", 3, "weights_of"), 7, "weights_of"),
                              (("layers", 2, "weights_of"), 1, "equal"),
                              (("layers", 2, "mixer", "scale"), 0.7, "equal"), (("norm",), None, "norm"),
                              (("layers", 1, "mlp", "kind"), "moe", "kind"), (("canon", "taps"), 0, "taps"), (("layers", 0, "mixer", "rot"), None, "rot")):
        with pytest.raises(ConfigError, match=word):
            config_from_dict(broken(path, value))


@pytest.mark.parametrize("name", list(CASES))
def test_the_model_declares_the_checkpoints_tensors(model_dirs, name):
    from glassbox_amd.config import config_from_dir
    from glassbox_amd.weights import SafetensorsFile
    from glassbox_amd.weights.loader import build_model, checkpoint_layout
    folder = folder_of(model_dirs.base, name)
    model = build_model(config_from_dir(folder))
    _, shapes = checkpoint_layout(model)
    f = SafetensorsFile(folder + "/model.safetensors")
    assert {n: tuple(f.shape(n)) for n in f.names()} == {n: tuple(s) for n, s in shapes.items()}
    raw = CASES[name]
    owners = [i for i, l in enumerate(raw["layers"]) if l.get("weights_of") is None]
    # tensors are numbered by the layer that owns them; a layer that borrows has none
    assert {int(n.split(".")[0][1:]) for n in shapes if n[0] == "l"} == set(owners)
    assert shapes["final.norm"] == () and all(shapes[f"l{i}.norm1"] == () for i in owners)
    assert ("l0.canon1" in shapes) == ("canon" in raw)
    # a cache layer (pages and state) of its own for every call, the block that of the owner
    assert [c.cache for c in model.schedule] == list(range(len(raw["layers"])))
    assert [owners[c.block] for c in model.schedule] == [pv.layer_owner(raw, i) for i in range(len(raw["layers"]))]
    states = model.state_specs()
    taps = raw.get("canon", {}).get("taps", 0)
    assert all((s is None) if taps < 2 else (s.shape == (taps - 1, raw["width"]) and s.dtype == torch.float32) for s in states)


def test_what_the_pages_hold():
    """Latent attention keeps every head's key [own part | shared rotated part] and value; differential attention one key
    head [map 1 | map 2] for the two maps of each query head of its group."""
    from glassbox_amd.parts.attention import DifferentialAttention, LatentAttention
    from glassbox_amd.parts.base import FULL, WINDOW
    m = LatentAttention(64, 4, 24, 8, 16, 24, 40, 0.4, window=24, rot_dims=8, rot_base=100.0)
    assert (m.cache_spec.num_kv_heads, m.cache_spec.head_dim, m.cache_spec.kind, m.cache_spec.window) == (4, 32, WINDOW, 24)
    assert LatentAttention(64, 2, 104, 32, 40, 8, 8, 0.1).cache_spec.head_dim == 136
    assert LatentAttention(64, 2, 16, 0, 40, 8, 8, 0.1).position is None
    d = DifferentialAttention(64, 4, 2, 16, 24, 0.5, 0.3, 0.4, 7)
    assert (d.cache_spec.num_kv_heads, d.cache_spec.head_dim, d.cache_spec.kind) == (2, 32, FULL)
    assert DifferentialAttention(64, 6, 1, 8, 48, 0.5, 0.3).cache_spec.head_dim == 48
    with pytest.raises(ValueError):
        LatentAttention(64, 2, 16, 8, 16, 8, 8, 0.1, rot_dims=10)
    with pytest.raises(ValueError):
        DifferentialAttention(64, 3, 2, 8, 8, 0.5, 0.3)


def test_a_model_with_state_refuses_shared_beginnings():
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.engine.engine import sharing_obstacles
    from glassbox_amd.weights.loader import build_model
    lines = sharing_obstacles(build_model(config_from_dict(CASES["A"])))
    assert any("state" in l for l in lines) and any("window" in l for l in lines)
