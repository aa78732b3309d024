"""The plain Taborax against properties that follow from its equations, and the configuration
reader and the spec of the engine's Taborax (no GPU)."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import plain_taborax as pt
from taborax_models import CONFIGS, MIXED, STRAIGHT, load_plain, make_folder
from tiny_models import random_tokens
from tokasaurus_amd.config.model_config import ConfigError
from tokasaurus_amd.config.taborax_config import ExpertsFF, TaboraxConfig
from tokasaurus_amd.models.registry import architecture_of, build_model


def test_unit_sink_is_one_more_score_of_zero():
    s = torch.randn(3, 5, 7, dtype=torch.float64) * 4
    p = pt.softmax_with_unit_sink(s)
    wider = torch.softmax(torch.cat([s, torch.zeros(3, 5, 1, dtype=torch.float64)], dim=-1), dim=-1)
    assert torch.allclose(p, wider[..., :-1], atol=1e-14)
    assert float(p.sum(-1).max()) < 1.0
    far_below = pt.softmax_with_unit_sink(torch.full((1, 4), -50.0, dtype=torch.float64))
    assert float(far_below.sum()) < 1e-20  # nothing but the sink: the output is next to nothing


def test_rotation_of_halves_depends_on_the_distance_only():
    rot = {"base": 100.0, "dims": 6}
    q, k = torch.randn(1, 1, 10, dtype=torch.float64), torch.randn(1, 1, 10, dtype=torch.float64)
    def dot(i, j):
        return float((pt.rotate_halves(q, torch.tensor([i]), rot) * pt.rotate_halves(k, torch.tensor([j]), rot)).sum())
    assert abs(dot(9, 4) - dot(105, 100)) < 1e-9 and abs(dot(9, 4) - dot(9, 5)) > 1e-6
    x = torch.randn(4, 2, 10, dtype=torch.float64)
    y = pt.rotate_halves(x, torch.arange(4), rot)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.equal(y[0], x[0])  # the rest passes; position 0 turns nothing
    # element i is paired with element i + 3: a turn of element 0 by a quarter lands in element 3
    e = torch.zeros(1, 1, 10, dtype=torch.float64)
    e[..., 0] = 1.0
    turned = pt.rotate_halves(e, torch.tensor([1]), {"base": 1.0, "dims": 6})
    assert abs(float(turned[0, 0, 0]) - math.cos(1.0)) < 1e-12 and abs(float(turned[0, 0, 3]) - math.sin(1.0)) < 1e-12


def test_latent_attention_is_attention_over_the_latent():
    """The form the engine computes: a head's query taken into the latent's space, one shared
    key/value head that is the latent, and the result taken to the head's values."""
    torch.manual_seed(0)
    T, W, H, d, dv, rq, r = 9, 12, 3, 4, 6, 5, 7
    mixer = {"heads": H, "dim": d, "vdim": dv, "q_rank": rq, "kv_rank": r, "scale": 0.3}
    shapes = {"dq": (rq, W), "dq.norm": (rq,), "uq": (H * d, rq), "dkv": (r, W), "dkv.norm": (r,), "uk": (H * d, r),
              "uv": (H * dv, r), "o": (W, H * dv)}
    w = {f"m.{k}": torch.randn(s, dtype=torch.float64) for k, s in shapes.items()}
    h = torch.randn(T, W, dtype=torch.float64)
    want = pt.latent_attention(h, w, "m", mixer, 1e-5)
    c = pt.norm(h @ w["m.dkv"].T, w["m.dkv.norm"], 1e-5)
    q = (pt.norm(h @ w["m.dq"].T, w["m.dq.norm"], 1e-5) @ w["m.uq"].T).view(T, H, d)
    q_lat = torch.einsum("thd,hdr->thr", q, w["m.uk"].view(H, d, r))
    s = (torch.einsum("ihr,jr->hij", q_lat, c) * 0.3).masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), -math.inf)
    o_lat = torch.einsum("hij,jr->ihr", torch.softmax(s, -1), c)
    o = torch.einsum("ihr,hvr->ihv", o_lat, w["m.uv"].view(H, dv, r)).reshape(T, H * dv)
    assert torch.allclose(o @ w["m.o"].T, want, atol=1e-10)


def test_router_groups_correction_and_weights():
    torch.manual_seed(1)
    W, E, I = 8, 6, 2
    w = {"f.router": torch.randn(E + I, W, dtype=torch.float64), "f.correction": torch.zeros(E + I, dtype=torch.float64)}
    h = torch.randn(40, W, dtype=torch.float64)
    s = torch.softmax(h @ w["f.router"].T, -1)
    # no groups, no correction: the plain top scores, their own values as weights (not summing to one)
    chosen, weight = pt.route(h, w, "f", {"experts": E, "identity": I, "top": 3})
    assert torch.equal(chosen, s.topk(3).indices) and torch.equal(weight, s.topk(3).values) and float(weight.sum(-1).max()) < 1
    # the correction moves the choice and not the weight; it may make choice scores negative
    w["f.correction"] = torch.tensor([-5.0] * 4 + [-1.0, -4.0, -2.5, -6.0], dtype=torch.float64)
    chosen, weight = pt.route(h, w, "f", {"experts": E, "identity": I, "top": 2})
    assert set(chosen.flatten().tolist()) <= {4, 6} and torch.equal(weight, s.gather(1, chosen))
    # groups of two neighbours, one kept: both choices come from the group of the best choice score,
    # though all choice scores are negative (a closed group counts as minus infinity, not as 0)
    chosen, _ = pt.route(h, w, "f", {"experts": E, "identity": I, "top": 2, "groups": {"count": 4, "keep": 1}})
    best = (s + w["f.correction"]).argmax(-1)
    assert torch.equal(chosen.min(-1).values // 2, best // 2) and torch.equal(chosen.max(-1).values // 2, best // 2)


def test_identity_experts_and_shared_expert():
    torch.manual_seed(2)
    W, F = 6, 4
    w = {"f.router": torch.zeros(3, W, dtype=torch.float64), "f.correction": torch.tensor([0.0, 0.0, 1.0], dtype=torch.float64)}
    for n, shape in (("gate", (F, W)), ("up", (F, W)), ("down", (W, F))):
        for e in ("e0", "e1", "shared"):
            w[f"f.{e}.{n}"] = torch.randn(shape, dtype=torch.float64)
    w["f.shared.sg"] = torch.randn(1, W, dtype=torch.float64)
    h = torch.randn(5, W, dtype=torch.float64)
    mlp = {"kind": "moe", "expert": {"ff": F}, "router": {"experts": 2, "identity": 1, "top": 1}}
    assert torch.allclose(pt.mixture_ff(h, w, "f", mlp), h / 3)  # the identity expert wins: its weight is the uniform score
    mlp["shared"] = {"ff": F}
    extra = pt.mixture_ff(h, w, "f", mlp) - h / 3
    assert torch.allclose(extra, torch.sigmoid(h @ w["f.shared.sg"].T) * pt.gated_expert(h, w, "f.shared"))


def test_run_order_and_the_first_layer_of_a_pass(tmp_path):
    assert pt.run_order({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert pt.run_order({"layers": [0] * 2}) == [0, 1]
    folder = make_folder(tmp_path / "m", MIXED, seed=1)
    cfg, w = load_plain(folder)
    tokens = random_tokens(11, cfg["vocab"], 3)
    streams = []
    logits = pt.forward(tokens, w, cfg, streams)
    assert len(streams) == 1 + 2 * 3 + 1 and logits.shape == (11, cfg["vocab"])
    # causal: a row does not depend on later tokens
    assert torch.allclose(pt.forward(tokens[:6], w, cfg), logits[:6], atol=1e-9)
    # the mixing matrix matters: without it the passes would differ
    w2 = dict(w)
    w2["loop.in"] = w["loop.in"] * 0.5
    assert float((pt.forward(tokens, w2, cfg) - logits).abs().max()) > 1e-3


def test_configuration_reader_and_spec():
    for name, raw in CONFIGS.items():
        arch = architecture_of(raw)
        assert arch.name == "taborax"
        cfg = arch.config_from_dict(raw)
        model = build_model(arch, cfg)
        order = [(e.layer, e.before is not None) for e in model.spec.run_order]
        assert [i for i, _ in order] == pt.run_order(raw)
        if raw.get("loop"):
            assert [first for i, first in order] == [i == raw["loop"]["start"] for i, _ in order]
        names = {s.name for s in model.tensor_specs()}
        assert ("loop.in" in names) == bool(raw.get("loop"))
        for i, layer in enumerate(raw["layers"]):
            assert (f"l{i}.norm2b" in names) == (layer["mlp"] is not None)
            assert (f"l{i}.mix.uk" in names) == (layer["type"] == "latent_attention")
            assert f"l{i}.mix.v" not in names
    cfg = TaboraxConfig.from_dict(STRAIGHT)
    ff = cfg.layers[0].ff
    assert isinstance(ff, ExpertsFF) and (ff.identity, ff.groups, ff.keep, ff.shared_ff) == (0, 3, 3, None)
    assert TaboraxConfig.from_dict(MIXED).layers[2].ff.groups == 1  # no groups given: one group, kept
    # every pass of a looped layer has a cache of its own: one need a run entry
    model = build_model(architecture_of(MIXED), TaboraxConfig.from_dict(MIXED))
    assert len(model.cache_needs()) == 8 and all(n is not None for n in model.cache_needs())
    assert model.cache_needs()[0].num_kv_heads == 1 and model.cache_needs()[0].head_dim == 48  # the latent alone is kept


@pytest.mark.parametrize("edit, message", [
    (lambda c: c["layers"][1]["mixer"].update(vdim=8), "values are the keys"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=34), "rotates"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "choices"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=5), "choices"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["layers"][0].update(type="recurrent"), "known"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "known"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_configuration_reader_refuses(edit, message):
    raw = copy.deepcopy(MIXED)
    edit(raw)
    with pytest.raises(ConfigError, match=message):
        TaboraxConfig.from_dict(raw)
