"""Tekilix without a device: the plain implementation pinned by what fixes it beside its own text, the configuration's
checks, the tensors the model declares, and the order of its layer calls."""
from __future__ import annotations

import copy
import math

import numpy as np
import pytest
import torch

from plain import tekilix as pt
from tekilix_cases import CASES, folder_of

F64 = torch.float64


# ------------------------------------------------------------------------------------------ the plain implementation
def test_the_bounded_norm_has_one_number_inside_and_a_weight_and_bias_outside():
    w = {"n": torch.tensor([2.0, -1.0], dtype=F64), "n.b": torch.tensor([0.5, 0.25], dtype=F64), "n.alpha": torch.tensor(3.0, dtype=F64)}
    out = pt.tanh_norm(w, "n", torch.tensor([[0.1, -0.2], [100.0, 0.0]], dtype=F64))
    assert out[0, 0] == pytest.approx(2.0 * math.tanh(0.3) + 0.5) and out[0, 1] == pytest.approx(-math.tanh(-0.6) + 0.25)
    assert out[1, 0] == pytest.approx(2.5) and out[1, 1] == pytest.approx(0.25)      # bounded, and no row statistic: rows are independent


def test_the_convolution_over_time_is_a_causal_correlation():
    torch.manual_seed(0)
    x, taps = torch.randn(11, 5, dtype=F64), torch.randn(5, 4, dtype=F64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.t()[None], (3, 0)), taps[:, None, :], groups=5)[0].t()
    assert torch.allclose(pt.causal_conv(x, taps), want, atol=1e-12)
    one = torch.zeros(6, 1, dtype=F64)
    one[2] = 1.0     # the last tap weighs the token itself, the first the oldest
    assert pt.causal_conv(one, torch.tensor([[1.0, 10.0, 100.0]], dtype=F64))[:, 0].tolist() == [0.0, 0.0, 100.0, 10.0, 1.0, 0.0]


@pytest.mark.parametrize("neighbours", [True, False])
def test_rotation_in_either_pairing_and_scores_that_depend_on_the_distance_alone(neighbours):
    rot = {"dims": 4, "base": 16.0}
    x = torch.zeros(3, 1, 6, dtype=F64)
    x[:, 0, 0] = 1.0                       # (1, 0) in the first pair: channels (0, 1) or (0, 2)
    x[:, 0, 5] = 7.0                       # beyond the rotated channels
    out = pt.rotate(x, torch.arange(3), rot, neighbours)
    partner = 1 if neighbours else 2
    for t in range(3):
        assert out[t, 0, 0] == pytest.approx(math.cos(t)) and out[t, 0, partner] == pytest.approx(math.sin(t))
        assert out[t, 0, 3 - partner] == 0.0 and out[t, 0, 5] == 7.0
    y = torch.zeros(2, 1, 4, dtype=F64)
    y[:, 0, 2 if neighbours else 1] = 1.0  # the second pair turns at base^(-2/4) a position
    got = pt.rotate(y, torch.tensor([0, 5]), rot, neighbours)
    assert got[1, 0, 2 if neighbours else 1] == pytest.approx(math.cos(5 / 4.0)) and got[1, 0, 3] == pytest.approx(math.sin(5 / 4.0))
    torch.manual_seed(1)
    q, k = torch.randn(1, 2, 8, dtype=F64).expand(9, 2, 8), torch.randn(1, 2, 8, dtype=F64).expand(9, 2, 8)
    rot = {"dims": 6, "base": 50.0, "scaling": {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}}
    rq, rk = pt.rotate(q, torch.arange(9), rot, neighbours), pt.rotate(k, torch.arange(9), rot, neighbours)
    assert torch.allclose((rq[5] * rk[2]).sum(-1), (rq[8] * rk[5]).sum(-1), atol=1e-12)
    assert not torch.allclose((rq[5] * rk[2]).sum(-1), (rq[5] * rk[4]).sum(-1), atol=1e-3)


def test_stretched_frequencies_by_hand():
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}}
    index = lambda turns: 8 * math.log(64 / (2 * math.pi * turns)) / (2 * math.log(100.0))
    lo, hi = max(math.floor(index(8.0)), 0), min(math.ceil(index(1.0)), 7)
    assert (lo, hi) == (0, 3)
    plain = [100.0 ** (-2 * i / 8) for i in range(4)]
    ramp = [min(max((i - lo) / (hi - lo), 0.0), 1.0) for i in range(4)]
    want = [f / 4.0 * r + f * (1 - r) for f, r in zip(plain, ramp)]
    got = pt.inverse_frequencies(rot)
    assert got.tolist() == pytest.approx(want) and got[0] == plain[0] and got[3] == pytest.approx(plain[3] / 4.0)
    assert pt.magnitude(rot) == pytest.approx(0.1 * math.log(4.0) + 1.0) and pt.magnitude({"dims": 8, "base": 100.0}) == 1.0
    # cosine and sine both carry the magnitude: a rotated vector is that much longer
    x = torch.ones(1, 1, 8, dtype=F64)
    assert float(pt.rotate(x, torch.tensor([3]), rot, False).norm()) == pytest.approx(pt.magnitude(rot) * math.sqrt(8.0))
    # the framework's table of frequencies is the same
    from glassbox_amd.parts.rotary import Rotary
    r = Rotary(8, 100.0, (4.0, 64, 8.0, 1.0))
    assert np.allclose(r.inv_host, np.array(want), rtol=1e-6) and r.magnitude == pytest.approx(pt.magnitude(rot))
    assert np.allclose(Rotary(8, 100.0).inv_host, np.array(plain), rtol=1e-6)


def test_visibility_in_runs_counted_from_the_first_position():
    see = pt.visible(12, 4)
    assert see[10, 10] and see[10, 8] and not see[10, 7] and not see[10, 11]
    assert see[8, 8] and not see[8, 7] and see[7, 4] and not see[7, 3]
    assert pt.visible(12)[11, 0] and not pt.visible(12)[3, 4]
    assert pt.visible(6, 1)[5, 5] and not pt.visible(6, 1)[5, 4]


def test_the_sink_takes_its_share_and_gives_nothing():
    torch.manual_seed(2)
    T, H = 7, 3
    s = torch.randn(H, T, T, dtype=F64)
    sink = torch.tensor([0.0, 2.0, -30.0], dtype=F64)
    p = pt.softmax_with_sink(s, pt.visible(T), sink)
    for h in range(H):
        for i in range(T):
            e = torch.exp(s[h, i, :i + 1])
            assert p[h, i, :i + 1].tolist() == pytest.approx((e / (e.sum() + math.exp(float(sink[h])))).tolist())
            assert float(p[h, i, i + 1:].abs().sum()) == 0.0
    assert float(p[2].sum(-1).min()) == pytest.approx(1.0) and float(p[1].sum(-1).max()) < 0.95
    assert float(pt.capped(torch.tensor(1000.0, dtype=F64), 25.0)) == pytest.approx(25.0)
    assert float(pt.capped(torch.tensor(0.5, dtype=F64), 25.0)) == pytest.approx(25.0 * math.tanh(0.02))
    assert float(pt.capped(torch.tensor(5.0, dtype=F64), 0.0)) == 5.0


def test_the_router_picks_by_corrected_scores_within_kept_groups_and_weighs_by_plain_ones():
    z = torch.tensor([[2.0, 1.9, 0.0, 0.1, 1.0, 1.1]], dtype=F64)
    s = torch.softmax(z, -1)
    none = torch.zeros(6, dtype=F64)
    ids, wts = pt.route(z, none, 2, None)
    assert sorted(ids[0].tolist()) == [0, 1] and wts[0].tolist() == pytest.approx([float(s[0, i]) for i in ids[0]])
    assert float(wts.sum()) < 1.0                                   # as they stand: not divided by their sum
    # groups (0,1) (2,3) (4,5): a group counts by its best expert; with one group kept both experts come from it
    ids, _ = pt.route(z, none, 2, {"count": 3, "keep": 1})
    assert sorted(ids[0].tolist()) == [0, 1]
    ids, _ = pt.route(z, none, 3, {"count": 3, "keep": 2})
    assert sorted(ids[0].tolist()) == [0, 1, 5]                     # the third comes from the second-best group, not expert 4's rival
    # the correction decides the choice (also the groups'), not the weights; it may be negative
    corr = torch.tensor([-1.0, -1.0, 0.0, 0.5, 0.0, 0.0], dtype=F64)
    ids, wts = pt.route(z, corr, 2, {"count": 3, "keep": 1})
    assert sorted(ids[0].tolist()) == [2, 3] and sorted(wts[0].tolist()) == pytest.approx(sorted([float(s[0, 2]), float(s[0, 3])]))
    ids, _ = pt.route(z, torch.full((6,), -5.0, dtype=F64), 2, {"count": 3, "keep": 1})
    assert sorted(ids[0].tolist()) == [0, 1]                        # negative picks are still above what was left out
    m = pt.route_margin(z, none, 2, None)
    assert float(m) == pytest.approx(float(s[0, 1] - s[0, 5]))
    assert math.isinf(float(pt.route_margin(z, none, 6, None)))


def test_the_experts_sum_is_the_weighted_sum_of_squared_relu_units_plus_the_shared_one():
    torch.manual_seed(3)
    d, E, ff = 6, 4, 5
    w = {f"m.e{e}.{n}": torch.randn(*(s), dtype=F64) for e in range(E) for n, s in (("up", (ff, d)), ("down", (d, ff)))}
    w.update({"m.router": torch.randn(E, d, dtype=F64), "m.correction": torch.randn(E, dtype=F64) * 0.1,
              "m.shared.up": torch.randn(3, d, dtype=F64), "m.shared.down": torch.randn(d, 3, dtype=F64)})
    mlp = {"router": {"experts": E, "top": 2, "groups": {"count": 2, "keep": 2}}, "shared": {"ff": 3}}
    x = torch.randn(9, d, dtype=F64)
    got = pt.experts(w, "m.", mlp, x)
    ids, wts = pt.route(x @ w["m.router"].T, w["m.correction"], 2, {"count": 2, "keep": 2})
    for t in range(9):
        want = w["m.shared.down"] @ torch.relu(w["m.shared.up"] @ x[t]) ** 2
        for e, a in zip(ids[t].tolist(), wts[t].tolist()):
            want = want + a * (w[f"m.e{e}.down"] @ torch.relu(w[f"m.e{e}.up"] @ x[t]) ** 2)
        assert torch.allclose(got[t], want, atol=1e-12)
    del mlp["shared"]
    assert not torch.allclose(pt.experts(w, "m.", mlp, x), got)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = str(tmp_path_factory.mktemp("tekilix"))
    return {name: folder_of(base, name) for name in CASES}


@pytest.mark.parametrize("name", list(CASES))
def test_every_layer_is_causal_and_reaches_as_far_as_its_run(folders, name):
    """Changing a token changes no logits before it; the logits at a later position change only if some layer's run of
    positions holds both (layers stack: a change can travel run by run only through tokens in between)."""
    cfg, w = pt.load_folder(folders[name])
    vocab = cfg["vocab"]
    torch.manual_seed(5)
    toks = torch.randint(0, vocab, (60,)).tolist()
    base = pt.forward(cfg, w, toks)
    at = 21
    other = list(toks)
    other[at] = (toks[at] + 1) % vocab
    moved = pt.forward(cfg, w, other)
    assert torch.allclose(moved[:at], base[:at], atol=1e-12) and not torch.allclose(moved[at], base[at], atol=1e-6)
    sizes = [(l["mixer"].get("mask") or {"size": 0})["size"] for l in cfg["layers"]]
    taps = max([l["mixer"].get("conv", 1) for l in cfg["layers"]])
    if all(sizes):
        # beyond the end of the longest run that holds the token (and the convolution's reach behind that), nothing moves
        end = max((at // s + 1) * s for s in sizes)
        reach = end
        for _ in cfg["layers"]:      # a change travels on through later layers: from any moved position to the end of its runs
            reach = max((min(reach + taps - 1, 59) // s + 1) * s for s in sizes) if reach < 60 else reach
        if reach < 60:
            assert torch.allclose(moved[reach + taps:], base[reach + taps:], atol=1e-12)
    else:
        assert not torch.allclose(moved[-1], base[-1], atol=1e-9)


def test_layers_that_use_anothers_tensors_are_that_layer_again(folders):
    cfg, w = pt.load_folder(folders["E"])
    assert [pt.layer_owner(cfg, i) for i in range(5)] == [0, 1, 0, 1, 0]
    written = copy.deepcopy(cfg)
    ww = dict(w)
    for i, layer in enumerate(written["layers"]):
        j = pt.layer_owner(cfg, i)
        layer.pop("weights_of", None)
        for k, v in w.items():
            if k.startswith(f"l{j}."):
                ww[f"l{i}." + k.split(".", 1)[1]] = v
    toks = list(range(3, 40))
    assert torch.allclose(pt.forward(cfg, w, toks), pt.forward(written, ww, toks), atol=1e-12)


# ------------------------------------------------------------------------------------------ configuration and model
def test_the_configuration_keeps_the_nested_keys_and_refuses_what_the_design_has_not():
    from glassbox_amd.config import ConfigError, config_from_dict
    for name, raw in CASES.items():
        cfg = config_from_dict(raw)
        assert cfg.architecture == "Tekilix" and config_from_dict(cfg.to_dict()) == cfg
    cfg = config_from_dict(CASES["E"])
    assert [cfg.owner(i) for i in range(5)] == [0, 1, 0, 1, 0] and cfg.embedding_scale == 5.0 and cfg.logit_scale == 0.25

    def broken(change):
        raw = copy.deepcopy(CASES["A"])
        change(raw)
        with pytest.raises(ConfigError):
            config_from_dict(raw)
    broken(lambda r: r["layers"][1]["mixer"].update(vdim=24))                      # the values are the keys
    broken(lambda r: r["layers"][0]["mixer"].update(kv_heads=3))
    broken(lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7))
    broken(lambda r: r["layers"][0]["mixer"]["rot"].update(scaling={"factor": 2.0, "original": 8, "fast": 2.0, "slow": 1.0}))
    broken(lambda r: r["layers"][0]["mlp"]["router"].update(top=7))
    broken(lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(count=4))     # six experts in four groups
    broken(lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(keep=1, count=6))   # one expert kept, two a token
    broken(lambda r: r["layers"][0]["mlp"].update(kind="dense"))
    broken(lambda r: r["layers"][2].update(weights_of=1))                           # another mixer than its own
    broken(lambda r: r["layers"][2].update(weights_of=2))
    broken(lambda r: r.pop("norm"))
    broken(lambda r: r["layers"][0].update(type="retention"))


def test_the_model_declares_the_checkpoints_tensors_and_one_cache_layer_a_call(folders):
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.engine.engine import check_supported
    from glassbox_amd.weights import SafetensorsFile
    from glassbox_amd.weights.loader import build_model, checkpoint_layout
    for name in CASES:
        model = build_model(config_from_dict(CASES[name]))
        _, shapes = checkpoint_layout(model)
        f = SafetensorsFile(folders[name] + "/model.safetensors")
        assert set(shapes) == set(f.names())
        f.close()
        layers = CASES[name]["layers"]
        assert len(model.schedule) == len(layers) and [c.cache for c in model.schedule] == list(range(len(layers)))
        assert len(model.blocks) == sum(1 for l in layers if l.get("weights_of") is None)
        for call, layer in zip(model.schedule, layers):
            spec, state = model.cache_specs()[call.cache], model.state_specs()[call.cache]
            m = layer["mixer"]
            assert spec.num_kv_heads == m["kv_heads"] and spec.head_dim >= max(m["dim"], m["vdim"])
            run = (m.get("mask") or {"size": 0})["size"]      # a layer that sees runs keeps the pages of the run at hand
            assert (spec.kind, spec.window) == ((2, run) if run else (0, 0))
            taps = m.get("conv", 0) if layer["type"] == "attention_2" else 0
            assert (state is None) == (taps <= 1)
            if state is not None:
                assert tuple(state.shape) == (taps - 1, (m["heads"] + m["kv_heads"]) * m["dim"])
        check_supported(model, torch.float32, 16)
        check_supported(model, torch.bfloat16, 16)
    names = set(checkpoint_layout(build_model(config_from_dict(CASES["A"])))[1])
    assert {"embed", "embed.norm", "embed.norm.b", "embed.norm.alpha", "l0.norm1", "l0.norm1b.b", "l0.norm2b.alpha", "l0.mix.q.b",
            "l0.mix.q.norm", "l0.mix.g", "l1.mix.q.conv", "l1.mix.sink", "l0.mlp.e5.up", "l0.mlp.correction", "l0.mlp.shared.down",
            "l4.norm1b", "final.norm", "final.norm.b"} <= names
    assert not {"l2.norm1", "l1.mix.v", "l1.mix.q.b", "l1.mlp.shared.up", "l4.norm2", "l0.mix.sink", "head"} & names
