"""Kupuzen through the engine against the plain model: every mechanism alone, prompts against
token-by-token decoding, portions down to two tokens, unequal requests in one batch on pages
and slots that are used again, keys just inside and just outside every window, long decoding,
and greedy generation through ``Engine.generate``."""

from __future__ import annotations

import copy
import json

import pytest
import torch

import plain_kupuzen as pk
from kupuzen_models import CONFIGS, MIXED, RECURRENT, TOL, WINDOWS, attention_layer, compare_rows, delta_layer, load_plain, make_folder, plain_rows
from replay_helpers import mixed_trace, portions, run_steps, tail_one_by_one, whole
from tiny_models import random_tokens
from tokasaurus_amd.engine.batch import StepEntry, layout, to_device
from tokasaurus_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu
PAGE = 16


@pytest.fixture(scope="module")
def kupuzen_folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("kupuzen")
    return {name: make_folder(root / name, cfg, seed=3 + i) for i, (name, cfg) in enumerate(sorted(CONFIGS.items()))}


def runner_for(folder, dtype, tokens=512, slots=4, **kw):
    return ModelRunner.from_folder(str(folder), dtype, page_size=PAGE, num_pages=tokens // PAGE, max_slots=slots, **kw)


def one_layer(layer: dict, width=64, vocab=120, **top) -> dict:
    cfg = {"architecture": "Kupuzen", "vocab": vocab, "width": width, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5},
           "residual_mult": 0.7, "layers": [layer]}
    cfg.update(top)
    return cfg


def streams_of(runner, tokens):
    """The residual stream after every block for one whole prompt."""
    planned = runner.plan([StepEntry("tap", tokens, [])])
    runner.storage.reset_slots(runner.manager.take_fresh_slots())
    hb = layout(planned, runner.model.spec.vocab_size, len(runner.groups), runner.manager.slot_tables)
    ctx, _, tables = to_device(hb, runner.model.dtype, runner.model.device, runner.storage.last_token)
    ctx.extras["kv_bound"] = runner.kv_bound(ctx.max_kv_len)
    tap: list = []
    ctx.extras["stream_tap"] = tap
    runner.model.forward(ctx, runner.cache_views(tables), runner.storage.states, None)
    runner.release("tap")
    return [t.cpu() for t in tap]


SINGLE_LAYERS = {
    "attention": attention_layer(4, 2, 16, 8, 0.3, window=7, rot={"base": 100.0, "dims": 6}),
    "attention_whole_rotation_no_window": attention_layer(3, 3, 8, 24, 0.5, rot={"base": 9.0, "dims": 8}, ff=40),
    "attention_matrix_core_sizes": attention_layer(8, 2, 40, 32, 0.3, window=19, rot={"base": 100.0, "dims": 10}),
    "attention_matrix_core_sizes_odd_group": attention_layer(6, 2, 8, 16, 0.3, rot={"base": 100.0, "dims": 8}),
    "delta": delta_layer(4, 2, 16, 24, 4, 8, 16),
    "delta_wide_key": delta_layer(2, 1, 136, 8, 2, 8, 8, ff=32),
    "delta_sizes_of_a_large_model": delta_layer(2, 1, 128, 128, 4, 16, 16),
    "delta_key_of_96": delta_layer(4, 4, 96, 64, 3, 8, 8),
    "attention_largest_heads_of_the_matrix_core_kernel": attention_layer(2, 1, 256, 256, 0.06, window=40, rot={"base": 1e4, "dims": 96}),
    "attention_heads_beyond_it": attention_layer(2, 2, 264, 16, 0.06, window=40, rot={"base": 1e4, "dims": 8}),
    "delta_largest_key": delta_layer(1, 1, 512, 16, 2, 8, 8),
    "attention_sizes_of_a_large_model": attention_layer(8, 2, 64, 64, 0.125, window=24, rot={"base": 500000.0, "dims": 64}),
    "feed_forward_beside_attention": attention_layer(1, 1, 8, 8, 1.0, window=2, ff=72),
}


@pytest.mark.parametrize("name", sorted(SINGLE_LAYERS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_alone(tmp_path, name, dtype):
    """A model of one layer: the stream after it and the logits, for a whole prompt."""
    config = one_layer(SINGLE_LAYERS[name], logit_softcap=5.0 if "delta" in name else None)
    folder = make_folder(tmp_path / name, config, seed=21)
    tokens = random_tokens(37, config["vocab"], 5)
    cfg, w = load_plain(folder)
    logits, streams = pk.forward(cfg, w, tokens, return_layers=True)
    runner = runner_for(folder, dtype, tokens=64)
    got = streams_of(runner, tokens)
    assert len(got) == 1 and got[0].dtype == torch.float32
    rel = float((got[0].double() - streams[0]).norm() / streams[0].norm())
    assert rel < (2e-5 if dtype == "float32" else 2e-2), f"stream after the layer: relative error {rel:.2e}"
    rows = run_steps(runner, whole("a", tokens))
    compare_rows(rows, {"a": logits.float()}, TOL[dtype])


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cutting_gives_the_plain_rows(kupuzen_folders, name, dtype):
    """Whole prompts, a tail decoded token by token (through recorded steps), portions of
    changing sizes down to two tokens and one, and unequal requests mixed in one batch on a
    pool so small that pages and slots are used again."""
    folder, vocab = kupuzen_folders[name], CONFIGS[name]["vocab"]
    reqs = {f"r{i}": random_tokens(n, vocab, 50 + i) for i, n in enumerate((70, 3, 41, 1, 97, 26))}
    plain = plain_rows(folder, reqs)
    runner = runner_for(folder, dtype, tokens=256)
    for rid, toks in reqs.items():
        compare_rows(run_steps(runner, whole(rid, toks)), plain, TOL[dtype])
    compare_rows(run_steps(runner, tail_one_by_one("r4", reqs["r4"], tail=40)), plain, TOL[dtype])
    compare_rows(run_steps(runner, portions("r4", reqs["r4"], [2, 3, 16, 2, 1, 31, 5])), plain, TOL[dtype])
    compare_rows(run_steps(runner, portions("r0", reqs["r0"], [15, 17, 1, 2])), plain, TOL[dtype])
    for seed in (1, 2):
        compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=4)), plain, TOL[dtype])
    assert runner.manager.requests == {}
    if dtype == "float32":
        # the same position from different cuttings: the same up to the order of 32-bit sums
        a = run_steps(runner, whole("r2", reqs["r2"]))
        b = run_steps(runner, portions("r2", reqs["r2"], [2, 7]))
        assert max(float((a[k] - b[k]).abs().max()) for k in a) < 2e-4


def test_batch_rows_do_not_depend_on_their_neighbours(kupuzen_folders):
    """A request alone and the same request between two others, as a prompt portion and as a
    single token: bit for bit the same logits in 32-bit (every kernel's order of sums is fixed
    by the token's own place; the batches are sized so that the 32-bit product, which has one
    form for few rows and one for many, takes the same form in both runs)."""
    folder, vocab = kupuzen_folders["mixed"], MIXED["vocab"]
    a, b, c = (random_tokens(n, vocab, 90 + n) for n in (33, 50, 19))
    runner = runner_for(folder, "float32", tokens=256)
    alone = run_steps(runner, [{"entries": [("b", b[:40], list(range(40)))]}, {"entries": [("b", b[40:41], [0])], "end": ["b"]}])
    beside = run_steps(runner, [
        {"entries": [("a", a[:20], []), ("b", b[:40], list(range(40))), ("c", c[:5], [])]},
        {"entries": [("a", a[20:21], []), ("b", b[40:41], [0]), ("c", c[5:6], [])], "end": ["a", "b", "c"]}])
    for key in alone:
        assert torch.equal(alone[key], beside[key]), f"{key} differs beside other requests"


def test_slots_and_pages_are_clean_for_their_next_holder(kupuzen_folders):
    """Two slots and a pool of eight pages serve six requests one after the other and in pairs:
    a request must not see the state or the keys of whoever held its slot and pages before."""
    folder, vocab = kupuzen_folders["mixed"], MIXED["vocab"]
    reqs = {f"q{i}": random_tokens(n, vocab, 70 + i) for i, n in enumerate((60, 64, 17, 49, 30, 5))}
    plain = plain_rows(folder, reqs)
    runner = runner_for(folder, "float32", tokens=128, slots=2)
    for seed in (3, 4):
        compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=2)), plain, TOL["float32"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_at_the_windows_edges_and_far_away(tmp_path, dtype):
    """One key is made to stand out: its token's key row and the last token's query row are
    scaled so that this one score dominates the softmax.  The logits then show whether that key
    is seen: the engine must agree with the plain model when the key lies just inside the
    window, just outside it, at a page's border, far back among hundreds, as a prompt's token
    and decoded alone."""
    window = 37
    layer = attention_layer(2, 1, 16, 16, 1.0, window=window, rot={"base": 20.0, "dims": 4})
    layer_all = attention_layer(2, 1, 16, 16, 1.0, rot={"base": 20.0, "dims": 4})
    config = one_layer(layer, width=32, vocab=64)
    config["layers"] = [layer, layer_all]
    config["layers"][1]["mixer"] = dict(layer_all["mixer"])
    folder = make_folder(tmp_path / "edges", config, seed=8, edits={
        # the sinks small, so that the one large score is not drowned
        ".sink": lambda t: t * 0.1 - 2.0})
    cfg, w = load_plain(folder)
    n = 300
    runner = runner_for(folder, dtype, tokens=320)
    worst = 0.0
    for back in (window - 1, window, 1, 15, 16, 17, 250):  # the marked key lies this far behind the last token
        tokens = random_tokens(n, 64, 100 + back)
        # token 63 appears once, at the marked place; its embedding is large, so its key is too
        tokens = [t % 63 for t in tokens]
        tokens[n - 1 - back] = 63
        w2 = dict(w)
        w2["embed"] = w["embed"].clone()
        plain = pk.forward(cfg, w2, tokens).float()
        for steps in (whole("e", tokens), tail_one_by_one("e", tokens, tail=3), portions("e", tokens, [2, 61])):
            got = run_steps(runner, steps)
            worst = max(worst, compare_rows({k: v for k, v in got.items() if k[1] >= n - 3}, {"e": plain}, TOL[dtype]))
    assert worst > 0


def test_a_marked_key_changes_the_logits_only_inside_the_window(tmp_path):
    """The plain model itself: with the marked key one step outside the window of the windowed
    layer the last row equals that of a prompt without the mark in that layer's view, so the
    test above does tell inside from outside."""
    layer = attention_layer(1, 1, 8, 8, 1.0, window=5)
    config = one_layer(layer, width=16, vocab=32)
    folder = make_folder(tmp_path / "mark", config, seed=2)
    cfg, w = load_plain(folder)
    base = random_tokens(20, 31, 4)
    inside, outside = list(base), list(base)
    inside[20 - 1 - 4] = 31
    outside[20 - 1 - 5] = 31
    ref = pk.forward(cfg, w, base)[-1]
    assert float((pk.forward(cfg, w, outside)[-1] - ref).abs().max()) < 1e-12
    assert float((pk.forward(cfg, w, inside)[-1] - ref).abs().max()) > 1e-3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(kupuzen_folders, dtype):
    """A short prompt and 400 tokens decoded one by one: the state is carried 400 times, the
    windows pass over decoded tokens and give their pages back."""
    folder, vocab = kupuzen_folders["mixed"], MIXED["vocab"]
    tokens = random_tokens(420, vocab, 77)
    plain = plain_rows(folder, {"d": tokens})
    runner = runner_for(folder, dtype, tokens=448)
    got = run_steps(runner, tail_one_by_one("d", tokens, tail=400))
    compare_rows(got, plain, TOL[dtype])
    assert all(step.captured for step in runner.recorded.values()) and runner.recorded


def test_first_tokens_of_a_sequence(kupuzen_folders):
    """Requests of one, two and three tokens, whole and token by token: the convolutions read
    zeros before the start, the state starts at zero, the windows are not full yet."""
    for name in ("mixed", "recurrent", "windows"):
        folder, vocab = kupuzen_folders[name], CONFIGS[name]["vocab"]
        reqs = {f"s{n}": random_tokens(n, vocab, 30 + n) for n in (1, 2, 3, 6)}
        plain = plain_rows(folder, reqs)
        runner = runner_for(folder, "float32", tokens=64)
        for rid, toks in reqs.items():
            compare_rows(run_steps(runner, whole(rid, toks)), plain, TOL["float32"])
            compare_rows(run_steps(runner, portions(rid, toks, [1])), plain, TOL["float32"])


@pytest.mark.parametrize("name", ["mixed", "recurrent"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(kupuzen_folders, dtype, name):
    """``Engine.generate``: the scheduler cuts prompts into portions beside decoding requests;
    the tokens are the plain model's greedy tokens (in bfloat16: each token is, for the plain
    logits of its own history, within rounding of the best)."""
    from tokasaurus_amd.config.engine_config import EngineConfig
    from tokasaurus_amd.engine.engine import Engine
    from tokasaurus_amd.sampling import SamplingParams

    folder, vocab = kupuzen_folders[name], CONFIGS[name]["vocab"]  # "recurrent" keeps no keys at all: no page is ever counted
    prompts = [random_tokens(n, vocab, 10 + n) for n in (5, 40, 23, 1, 64)]
    engine = Engine(EngineConfig(model=str(folder), dtype=dtype, page_size=PAGE, kv_cache_num_tokens=512, max_seqs_per_forward=3,
                                 max_tokens_per_forward=24, allocator_sanity_checks=True))
    done = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    cfg, w = load_plain(folder)
    for prompt, c in zip(prompts, done):
        assert len(c.tokens) == 12 and c.finish_reason == "length"
        ids = list(prompt)
        for tok in c.tokens:
            logits = pk.forward(cfg, w, ids)[-1]
            if dtype == "float32":
                assert tok == int(logits.argmax()), f"token {tok}, plain {int(logits.argmax())}"
            else:
                assert float(logits.max() - logits[tok]) < 0.05 * float(logits.std()) + 0.05
            ids.append(tok)
    assert engine.runner.manager.requests == {}


def test_command_line_and_trace_replay(kupuzen_folders, tmp_path):
    """``bin/toka`` generates from a Kupuzen folder (also from a config.json alone, with random weights, where the
    low ranks that no checkpoint gives come from the file or a default), and ``bin/trace_run`` replays given tokens
    step by step: its logits are the plain model's."""
    import os
    import subprocess
    import sys

    import numpy as np

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, vocab = kupuzen_folders["mixed"], MIXED["vocab"]
    prompts = [random_tokens(9, vocab, 1), random_tokens(20, vocab, 2)]
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "toka"), f"model={folder}", "dtype=float32", f"page_size={PAGE}",
                           "kv_cache_num_tokens=256", f"prompt_ids=({json.dumps(prompts)})", "max_tokens=5", "ignore_eos=T"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [json.loads(l) for l in proc.stdout.splitlines() if l.strip()]
    cfg, w = load_plain(folder)
    for prompt, line in zip(prompts, lines):
        ids = list(prompt)
        for tok in line["tokens"]:
            assert tok == int(pk.forward(cfg, w, ids)[-1].argmax())
            ids.append(tok)
    bare = copy.deepcopy(RECURRENT)
    for layer in bare["layers"]:
        del layer["mixer"]["decay_rank"], layer["mixer"]["gate_rank"]
    model = tmp_path / "fresh"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(bare))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "toka"), f"model={model}", "random_weights=T", "seed=5",
                           "dtype=bfloat16", "num_prompts=2", "prompt_len=7", "max_tokens=3"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert (model / "model.safetensors").is_file() and len(proc.stdout.splitlines()) == 2
    # the replay tool: two requests, portions beside single tokens, the first ended before the second
    a, b = random_tokens(21, vocab, 3), random_tokens(40, vocab, 4)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": [0]}, {"id": "b", "tokens": b[:33], "want": [32]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[33:35], "want": []}, {"id": "a", "tokens": a[18:], "want": [2]}], "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b[35:], "want": [4]}], "end": ["b"]},
    ]
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(folder), "--dtype", "float32",
                           "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    plain = plain_rows(folder, {"a": a, "b": b})
    want = {0: [("a", 0), ("a", 16)], 1: [("a", 17), ("b", 32)], 2: [("a", 20)], 3: [("b", 39)]}
    for step, rows in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(rows), vocab).copy())
        compare_rows({key: got[i] for i, key in enumerate(rows)}, plain, TOL["float32"])
