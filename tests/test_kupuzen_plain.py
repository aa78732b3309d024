"""Runs without a GPU: the plain Kupuzen's mechanisms against properties that follow from
their equations, the configuration reader, and how the model is put together from parts."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import plain_kupuzen as pk
from kupuzen_models import CONFIGS, MIXED, RECURRENT, WINDOWS
from tokasaurus_amd.cache.manager import plan_groups
from tokasaurus_amd.config.kupuzen_config import KupuzenConfig
from tokasaurus_amd.config.model_config import ConfigError
from tokasaurus_amd.models.registry import architecture_of, build_model
from tokasaurus_amd.parts.position import interleaved_frequencies


def test_frequencies_follow_the_three_bands():
    rot = {"base": 10000.0, "dims": 16, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 32}}
    plain = pk.rotary_frequencies(rot)
    base = torch.tensor([10000.0 ** (-2.0 * i / 16) for i in range(8)], dtype=torch.float64)
    wavelength = 2 * math.pi / base
    assert bool((plain[wavelength < 8] == base[wavelength < 8]).all())
    assert torch.allclose(plain[wavelength > 32], base[wavelength > 32] / 8.0)
    mid = (wavelength >= 8) & (wavelength <= 32)
    assert bool(mid.any()) and bool(((plain[mid] < base[mid]) & (plain[mid] > base[mid] / 8.0)).all())
    engine = interleaved_frequencies(16, 10000.0, rot["scaling"])
    assert engine.dtype == torch.float32 and torch.allclose(engine.double(), plain, rtol=1e-7)
    assert torch.equal(interleaved_frequencies(6, 50.0, None).double(),
                       torch.tensor([1.0, 50.0 ** (-2 / 6), 50.0 ** (-4 / 6)], dtype=torch.float64).float().double())


def test_rotation_pairs_neighbours_and_leaves_the_rest():
    x = torch.randn(3, 2, 10, dtype=torch.float64)
    f = torch.tensor([1.0, 0.5], dtype=torch.float64)
    pos = torch.tensor([0, 1, 7])
    y = pk.rotate_interleaved(x, pos, f)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 4:], x[..., 4:])
    # a rotation keeps every pair's length and depends on the position difference only
    assert torch.allclose(y[..., 0:2].norm(dim=-1), x[..., 0:2].norm(dim=-1))
    q, k = torch.randn(1, 1, 4, dtype=torch.float64), torch.randn(1, 1, 4, dtype=torch.float64)
    d = [float((pk.rotate_interleaved(q, torch.tensor([p + 3]), f) * pk.rotate_interleaved(k, torch.tensor([p]), f)).sum()) for p in (0, 5, 40)]
    assert abs(d[0] - d[1]) < 1e-12 and abs(d[0] - d[2]) < 1e-12


def test_short_convolution_is_causal_with_the_last_tap_on_the_current_token():
    x = torch.zeros(6, 1, dtype=torch.float64)
    x[2] = 1.0
    taps = torch.tensor([[0.1, 0.2, 0.3, 0.4]], dtype=torch.float64)
    assert pk.short_conv(x, taps)[:, 0].tolist() == [0.0, 0.0, 0.4, 0.3, 0.2, 0.1]


def _delta_weights(H, G, dk, dv, width, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    p = "m"
    w = {f"{p}.q": r(G * dk, width), f"{p}.k": r(G * dk, width), f"{p}.v": r(H * dv, width),
         f"{p}.q.conv": r(G * dk, 3), f"{p}.k.conv": r(G * dk, 3), f"{p}.v.conv": r(H * dv, 3),
         f"{p}.b": r(H, width), f"{p}.a1": r(4, width), f"{p}.a2": r(H * dk, 4), f"{p}.g1": r(4, width),
         f"{p}.g2": r(H * dv, 4), f"{p}.o": r(width, H * dv), f"{p}.A_log": r(H), f"{p}.dt_bias": r(H * dk),
         f"{p}.norm": r(dv)}
    return w


def test_delta_rule_with_no_decay_and_full_strength_recalls_the_value_it_wrote():
    """With g = 1 and beta = 1 a token whose key was never seen before (orthogonal to the
    earlier keys) is stored exactly: S^T k = v right after its write."""
    dk, dv = 4, 3
    S = torch.zeros(dk, dv, dtype=torch.float64)
    keys = torch.eye(dk, dtype=torch.float64)
    vals = torch.randn(dk, dv, dtype=torch.float64)
    for t in range(dk):
        u = 1.0 * (vals[t] - S.T @ keys[t])
        S = S + torch.outer(keys[t], u)
    for t in range(dk):
        assert torch.allclose(S.T @ keys[t], vals[t])
    # and the plain mixer is causal: a later token does not change earlier outputs
    mixer = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 3, "conv": 3}
    w = _delta_weights(2, 1, 4, 3, 5, 1)
    h = torch.randn(7, 5, dtype=torch.float64)
    full = pk.channel_delta(h, w, "m", mixer, 1e-6)
    assert torch.allclose(pk.channel_delta(h[:4], w, "m", mixer, 1e-6), full[:4])


def test_sink_takes_its_share_and_window_counts_the_token_itself():
    mixer = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 1.0, "mask": {"size": 2}, "rot": {"base": 10.0, "dims": 0}}
    T = 4
    w = {"m.q": torch.zeros(2, 2, dtype=torch.float64), "m.q.norm": torch.ones(2, dtype=torch.float64),
         "m.sink": torch.tensor([0.0], dtype=torch.float64), "m.o": torch.ones(1, 1, dtype=torch.float64)}
    k = torch.zeros(T, 1, 2, dtype=torch.float64)
    v = torch.arange(1.0, T + 1, dtype=torch.float64).view(T, 1, 1)
    out, _ = pk.attention(torch.zeros(T, 2, dtype=torch.float64), w, "m", mixer, 1e-6, torch.arange(T), kv=(k, v))
    # all scores are 0 = the sink: position 0 sees itself (weight 1/2), later ones two keys (1/3 each)
    assert torch.allclose(out[:, 0], torch.tensor([1 / 2, (1 + 2) / 3, (2 + 3) / 3, (3 + 4) / 3], dtype=torch.float64))


def test_configuration_reader_names_what_is_missing_or_unknown():
    cfg = KupuzenConfig.from_dict(MIXED)
    assert len(cfg.layers) == 5 and cfg.layers[2].mixer.kv_from == 0 and cfg.layers[4].mixer.window == 0
    assert cfg.layers[1].ff is None and cfg.layers[1].mixer.decay_rank == 12 and cfg.logit_softcap == 8.0
    assert KupuzenConfig.from_dict(RECURRENT).logit_softcap is None
    bad = copy.deepcopy(MIXED)
    del bad["layers"][0]["mixer"]["scale"]
    with pytest.raises(ConfigError, match=r"layers\[0\].mixer lacks 'scale'"):
        KupuzenConfig.from_dict(bad)
    bad = copy.deepcopy(MIXED)
    bad["layers"][1]["type"] = "something"
    with pytest.raises(ConfigError, match="known: attention, channel_delta"):
        KupuzenConfig.from_dict(bad)
    bad = copy.deepcopy(MIXED)
    bad["layers"][2]["mixer"]["kv_from"] = 1
    with pytest.raises(ConfigError, match="no earlier attention layer"):
        KupuzenConfig.from_dict(bad)
    bad = copy.deepcopy(MIXED)
    bad["layers"][2]["mixer"]["dim"] = 32
    with pytest.raises(ConfigError, match="differ in head layout"):
        KupuzenConfig.from_dict(bad)
    # ranks that the file does not give come from the checkpoint's shapes
    bare = copy.deepcopy(MIXED)
    del bare["layers"][1]["mixer"]["decay_rank"], bare["layers"][1]["mixer"]["gate_rank"]
    cfg = KupuzenConfig.from_dict(bare).with_tensor_shapes({"l1.mix.a1": (10, 96), "l1.mix.g1": (6, 96)})
    assert (cfg.layers[1].mixer.decay_rank, cfg.layers[1].mixer.gate_rank) == (10, 6)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_model_is_put_together_from_the_file_alone(name):
    config = CONFIGS[name]
    arch = architecture_of(config)
    assert arch.name == "kupuzen"
    model = build_model(arch, arch.config_from_dict(config))
    specs = {s.name: s.shape for s in model.tensor_specs()}
    for i, layer in enumerate(config["layers"]):
        m = layer["mixer"]
        assert specs[f"l{i}.norm1"] == (config["width"],)
        assert (f"l{i}.norm2" in specs) == (layer["mlp"] is not None) == (f"l{i}.mlp.down" in specs)
        assert specs[f"l{i}.mix.o"] == (config["width"], m["heads"] * m["vdim"])
        if layer["type"] == "attention":
            assert specs[f"l{i}.mix.sink"] == (m["heads"],) and specs[f"l{i}.mix.q.norm"] == (m["heads"] * m["dim"],)
            assert (f"l{i}.mix.k" in specs) == ("kv_from" not in m) == (f"l{i}.mix.k.norm" in specs) == (f"l{i}.mix.v" in specs)
        else:
            assert specs[f"l{i}.mix.a2"] == (m["heads"] * m["dim"], m["decay_rank"])
            assert specs[f"l{i}.mix.q.conv"] == (m["kv_heads"] * m["dim"], m["conv"])
            assert specs[f"l{i}.mix.dt_bias"] == (m["heads"] * m["dim"],) and specs[f"l{i}.mix.norm"] == (m["vdim"],)
    assert specs["head"] == (config["vocab"], config["width"]) and specs["embed"] == specs["head"]


def test_a_cache_that_another_layer_reads_keeps_the_wider_window():
    arch = architecture_of(MIXED)
    model = build_model(arch, arch.config_from_dict(MIXED))
    needs = model.cache_needs()
    assert needs[0].window == 21 and needs[2].window == 21 and needs[4].window == 0 and needs[1] is None
    assert needs[0].value_size == 16 and needs[4].value_dim == 0
    groups, where = plan_groups(needs, [e.cache_of for e in model.spec.run_order])
    assert len(groups) == 2 and where[0] == where[2] and where[1] is None
    assert [s is not None for s in model.state_needs()] == [False, True, False, True, False]
    arch = architecture_of(WINDOWS)
    needs = build_model(arch, arch.config_from_dict(WINDOWS)).cache_needs()
    assert [n.window for n in needs] == [1, 11, 16, 16, 64]
