"""Taborax through the engine against the plain model: every mechanism alone, prompts against
token-by-token decoding, portions down to two tokens, unequal requests in one batch on pages
and slots that are used again, keys far back and at page borders, first tokens, long decoding,
and greedy generation through ``Engine.generate``."""

from __future__ import annotations

import json

import pytest
import torch

import plain_taborax as pt
from taborax_models import (CONFIGS, MIXED, STEADY, TOL, attention_layer, compare_rows, dense, latent_layer, load_plain, make_folder,
                            moe, plain_rows)
from replay_helpers import mixed_trace, portions, run_steps, tail_one_by_one, whole
from tiny_models import random_tokens
from tokasaurus_amd.engine.batch import StepEntry, layout, to_device
from tokasaurus_amd.engine.runner import ModelRunner
from tokasaurus_amd.kernels import ops

pytestmark = pytest.mark.gpu
PAGE = 16


@pytest.fixture(scope="module")
def taborax_folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("taborax")
    return {(name, steady): make_folder(root / f"{name}{int(steady)}", cfg, seed=5 + i, steady_choice=steady)
            for i, (name, cfg) in enumerate(sorted(CONFIGS.items())) for steady in (False, True)}


def runner_for(folder, dtype, tokens=512, slots=4, **kw):
    return ModelRunner.from_folder(str(folder), dtype, page_size=PAGE, num_pages=tokens // PAGE, max_slots=slots, **kw)


def one_layer(layer: dict, width=64, vocab=120, **top) -> dict:
    cfg = {"architecture": "Taborax", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "layers": [layer]}
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


# ---------------------------------------------------------------------------------- kernels alone


def test_router_kernel_against_the_plain_router():
    """Scores, groups, correction, choice and weights, for sizes with and without groups, more
    experts than a wavefront has lanes, and one choice."""
    torch.manual_seed(3)
    for n_all, identity, groups, keep, top, width in ((12, 2, 4, 2, 3, 40), (5, 0, 1, 1, 1, 24), (130, 2, 10, 3, 8, 64), (6, 6, 3, 1, 2, 8)):
        w = {"f.router": (torch.randn(n_all, width) * 0.6).bfloat16().double(), "f.correction": (torch.randn(n_all) * 0.05).bfloat16().double()}
        h = torch.randn(70, width).bfloat16().double()
        router = {"experts": n_all - identity, "identity": identity, "top": top, "groups": {"count": groups, "keep": keep}}
        chosen, weight = pt.route(h, w, "f", router)
        gate_w = torch.randn(width).bfloat16()
        for dtype in (torch.float32, torch.bfloat16):
            ids, wts, gate = ops.expert_route(h.to(dtype).cuda(), w["f.router"].to(dtype).cuda(), w["f.correction"].float().cuda(),
                                              groups, keep, top, gate_w.to(dtype).cuda())
            assert torch.equal(ids.cpu().long(), chosen), f"{n_all} experts in {groups} groups"
            assert torch.allclose(wts.cpu().double(), weight, atol=1e-6)
            assert torch.allclose(gate.cpu().double(), torch.sigmoid(h @ gate_w.double()), atol=1e-5)


@pytest.mark.parametrize("T, E, W, F, top", [(9, 5, 24, 12, 3), (70, 5, 24, 16, 3), (150, 7, 40, 72, 2), (33, 40, 64, 8, 4)])
def test_expert_kernels_against_plain_experts(T, E, W, F, top):
    """The chosen experts' weighted sum with identity experts, an empty place and a shared expert: pair by pair
    for few tokens, sorted by expert into tiles on the matrix cores for many (bfloat16); experts that no token
    chose, experts with more pairs than a tile holds."""
    torch.manual_seed(4)
    w = {}
    for e in range(E):
        w.update({f"f.e{e}.gate": torch.randn(F, W) / 5, f"f.e{e}.up": torch.randn(F, W) / 5, f"f.e{e}.down": torch.randn(W, F) / 3})
    w = {k: v.bfloat16().double() for k, v in w.items()}
    h = torch.randn(T, W).bfloat16().double()
    ids = torch.randint(0, E + 2, (T, top), dtype=torch.int32)
    ids[ids == 1] = 0  # nobody chooses expert 1; expert 0 gets many
    ids[0, 1] = -1
    wts = torch.rand(T, top)
    shared, gate = torch.randn(T, W), torch.rand(T)
    want = shared.double() * gate.double()[:, None]
    for t in range(T):
        for k in range(top):
            e = int(ids[t, k])
            if e >= 0:
                want[t] += wts[t, k].double() * (pt.gated_expert(h[t : t + 1], w, f"f.e{e}")[0] if e < E else h[t])
    gu = torch.stack([torch.cat([w[f"f.e{e}.gate"], w[f"f.e{e}.up"]]) for e in range(E)])
    dn = torch.stack([w[f"f.e{e}.down"] for e in range(E)])
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
        got = ops.expert_mix(h.to(dtype).cuda(), gu.to(dtype).cuda(), dn.to(dtype).cuda(), ids.cuda(), wts.cuda(), shared.cuda(), gate.cuda())
        rel = (got.cpu().double() - want).norm(dim=-1) / want.norm(dim=-1)
        assert float(rel.max()) < tol, f"{dtype}: rows {torch.nonzero(rel > tol).flatten().tolist()[:8]} of {T}"


def test_head_linear_and_stream_kernels():
    torch.manual_seed(5)
    x, w = torch.randn(7, 3 * 10 + 2), torch.randn(3, 6, 10)
    want = torch.einsum("thi,hoi->tho", x[:, :30].view(7, 3, 10).double(), w.double()).reshape(7, 18)
    assert torch.allclose(ops.head_linear(x.cuda(), w.cuda()).cpu().double(), want, atol=1e-5)
    got16 = ops.head_linear(x.bfloat16().cuda(), w.bfloat16().cuda(), out_f32=True).cpu().double()
    assert got16.dtype == torch.float64 and float((got16 - want).abs().max()) < 0.2
    # many rows: tiles on the matrix cores; inner sizes that end inside a step of 32, outputs that end inside a block of 16
    for rows, heads, n_in, n_out in ((50, 3, 40, 24), (33, 2, 64, 100), (200, 5, 8, 16), (17, 1, 72, 7)):
        x, w = torch.randn(rows, heads * n_in).bfloat16(), torch.randn(heads, n_out, n_in).bfloat16()
        want = torch.einsum("thi,hoi->tho", x.view(rows, heads, n_in).double(), w.double()).reshape(rows, heads * n_out)
        got = ops.head_linear(x.cuda(), w.cuda(), out_f32=True).cpu().double()
        assert float((got - want).abs().max()) < 1e-3 * n_in ** 0.5, (rows, heads, n_in, n_out)
        got = ops.head_linear(x.cuda(), w.cuda()).cpu().double()
        assert float((got - want).abs().max()) < 0.05 * n_in ** 0.5
    for width in (96, 100, 37):  # rows held in registers, and read back
        s, a = torch.randn(5, width), torch.randn(5, width) * 3
        wb, wn = torch.rand(width) + 0.5, torch.rand(width) + 0.5
        new = s.double() + pt.norm(a.double(), wb.double(), 1e-5)
        x_new, h = ops.post_norm_residual(s.cuda(), a.cuda(), wb.cuda(), 1e-5, wn.cuda(), 1e-3, torch.float32, in_place=False)
        assert torch.allclose(x_new.cpu().double(), new, atol=1e-5)
        assert torch.allclose(h.cpu().double(), pt.norm(new, wn.double(), 1e-3), atol=1e-5)
        both = ops.concat_cast(s.cuda(), a.cuda(), torch.bfloat16).cpu()
        assert torch.equal(both, torch.cat([s, a], dim=1).bfloat16())
    y = torch.randn(33)
    assert torch.allclose(ops.squared_relu_(y.clone().cuda()).cpu(), torch.relu(y) ** 2)


# ---------------------------------------------------------------------------------- every mechanism as a model of one layer

SINGLE_LAYERS = {
    "latent": latent_layer(4, 16, 24, 20, 32, 0.25),
    "latent_one_head_odd_sizes": latent_layer(1, 12, 7, 9, 21, 0.3),
    "latent_sizes_of_a_large_model": latent_layer(8, 64, 96, 72, 192, 0.12, dense(96)),
    "latent_beyond_the_matrix_core_kernel": latent_layer(2, 16, 16, 24, 272, 0.1),
    "latent_more_heads_than_the_plain_kernel_takes_at_once": latent_layer(9, 8, 16, 16, 264, 0.1),
    "attention_halves_of_a_part": attention_layer(4, 2, 32, 0.18, rot={"base": 100.0, "dims": 12}),
    "attention_whole_head_no_grouping": attention_layer(3, 3, 8, 0.4, rot={"base": 9.0, "dims": 8}),
    "attention_no_rotation_odd_head": attention_layer(6, 1, 14, 0.3),
    "attention_sizes_of_a_large_model": attention_layer(8, 2, 128, 0.09, rot={"base": 500000.0, "dims": 64}),
    "dense": attention_layer(1, 1, 8, 1.0, mlp=dense(72)),
    "experts_groups_identity_shared": attention_layer(1, 1, 8, 1.0, mlp=moe(24, 13, 4, identity=3, groups=(4, 3), shared=16)),
    "experts_one_choice": latent_layer(1, 8, 8, 8, 8, 0.5, moe(40, 3, 1)),
    "experts_only_identity_chosen_often": attention_layer(1, 1, 8, 1.0, mlp=moe(8, 2, 2, identity=4, groups=(3, 2))),
}


@pytest.mark.parametrize("name", sorted(SINGLE_LAYERS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_layer_alone(tmp_path, name, dtype):
    """A model of one layer: the stream after it and the logits, for a whole prompt."""
    config = one_layer(SINGLE_LAYERS[name])
    folder = make_folder(tmp_path / name, config, seed=21, steady_choice=STEADY[dtype])
    tokens = random_tokens(37, config["vocab"], 5)
    cfg, w = load_plain(folder)
    streams: list = []
    logits = pt.forward(tokens, w, cfg, streams)
    runner = runner_for(folder, dtype, tokens=64)
    got = streams_of(runner, tokens)
    assert len(got) == 1 and got[0].dtype == torch.float32
    rel = (got[0].double() - streams[0]).norm(dim=-1) / streams[0].norm(dim=-1)
    whole_rel = float((got[0].double() - streams[0]).norm() / streams[0].norm())
    assert whole_rel < (2e-5 if dtype == "float32" else 2e-2), f"stream after the layer: relative error {whole_rel:.2e}"
    assert float(rel.max()) < (5e-5 if dtype == "float32" else 6e-2), f"stream after the layer, row by row: {rel.tolist()}"
    compare_rows(run_steps(runner, whole("a", tokens)), {"a": logits.float()}, TOL[dtype])


# ---------------------------------------------------------------------------------- cuttings, batches, reuse


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_every_cutting_gives_the_plain_rows(taborax_folders, name, dtype):
    """Whole prompts, a tail decoded token by token (through recorded steps), portions of
    changing sizes down to two tokens and one, and unequal requests mixed in one batch on a
    pool so small that pages and slots are used again."""
    folder, vocab = taborax_folders[name, STEADY[dtype]], CONFIGS[name]["vocab"]
    reqs = {f"r{i}": random_tokens(n, vocab, 50 + i) for i, n in enumerate((70, 3, 41, 1, 97, 26))}
    plain = plain_rows(folder, reqs)
    runner = runner_for(folder, dtype, tokens=256)
    tol, flips = TOL[dtype], 0.0
    for rid, toks in reqs.items():
        compare_rows(run_steps(runner, whole(rid, toks)), plain, tol, flips)
    compare_rows(run_steps(runner, tail_one_by_one("r4", reqs["r4"], tail=40)), plain, tol, flips)
    compare_rows(run_steps(runner, portions("r4", reqs["r4"], [2, 3, 16, 2, 1, 31, 5])), plain, tol, flips)
    compare_rows(run_steps(runner, portions("r0", reqs["r0"], [15, 17, 1, 2])), plain, tol, flips)
    for seed in (1, 2):
        compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=4)), plain, tol, flips)
    assert runner.manager.requests == {}
    if dtype == "float32":
        # the same position from different cuttings: the same up to the order of 32-bit sums
        a = run_steps(runner, whole("r2", reqs["r2"]))
        b = run_steps(runner, portions("r2", reqs["r2"], [2, 7]))
        assert max(float((a[k] - b[k]).abs().max()) for k in a) < 2e-4


def test_batch_rows_do_not_depend_on_their_neighbours(taborax_folders):
    """A request alone and the same request between two others, as a prompt portion and as a
    single token: bit for bit the same logits in 32-bit (every kernel's order of sums is fixed
    by the token's own place; the batches are sized so that the 32-bit product, which has one
    form for few rows and one for many, takes the same form in both runs)."""
    folder, vocab = taborax_folders["mixed", False], MIXED["vocab"]
    a, b, c = (random_tokens(n, vocab, 90 + n) for n in (33, 50, 19))
    runner = runner_for(folder, "float32", tokens=256)
    alone = run_steps(runner, [{"entries": [("b", b[:40], list(range(40)))]}, {"entries": [("b", b[40:41], [0])], "end": ["b"]}])
    beside = run_steps(runner, [
        {"entries": [("a", a[:20], []), ("b", b[:40], list(range(40))), ("c", c[:5], [])]},
        {"entries": [("a", a[20:21], []), ("b", b[40:41], [0]), ("c", c[5:6], [])], "end": ["a", "b", "c"]}])
    for key in alone:
        assert torch.equal(alone[key], beside[key]), f"{key} differs beside other requests"


def test_slots_and_pages_are_clean_for_their_next_holder(taborax_folders):
    """Two slots and a pool of eight pages a group serve six requests one after the other and
    in pairs: a request must not see the keys of whoever held its pages before."""
    folder, vocab = taborax_folders["mixed", False], MIXED["vocab"]
    reqs = {f"q{i}": random_tokens(n, vocab, 70 + i) for i, n in enumerate((60, 64, 17, 49, 30, 5))}
    plain = plain_rows(folder, reqs)
    runner = runner_for(folder, "float32", tokens=128, slots=2)
    for seed in (3, 4):
        compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=2)), plain, TOL["float32"])


@pytest.mark.parametrize("kind", ["latent", "attention"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_key_far_back_and_at_page_borders(tmp_path, dtype, kind):
    """One key is made to stand out: its token appears once and its embedding is large, so the
    last tokens' scores for it dominate the softmax.  The logits then show whether that key is
    read from the right place: one token back, at both sides of a page's border, and far back
    among hundreds, in a prompt's portion and decoded alone."""
    layer = latent_layer(2, 16, 16, 16, 32, 1.0) if kind == "latent" else attention_layer(2, 1, 16, 1.0, rot={"base": 20.0, "dims": 4})
    config = one_layer(layer, width=32, vocab=64)
    config["layers"] = [layer, json.loads(json.dumps(layer))]
    folder = make_folder(tmp_path / "marked", config, seed=8, edits={"embed": lambda t: torch.cat([t[:63], t[63:] * 6.0])})
    cfg, w = load_plain(folder)
    n = 300
    runner = runner_for(folder, dtype, tokens=320)
    changed = 0.0
    for back in (1, 15, 16, 17, 31, 32, 250, 299):  # the marked key lies this far behind the last token
        tokens = [t % 63 for t in random_tokens(n, 64, 100 + back)]
        unmarked = pt.forward(tokens, w, cfg)[-1]
        tokens[n - 1 - back] = 63
        plain = pt.forward(tokens, w, cfg).float()
        changed = max(changed, float((plain[-1] - unmarked).abs().max()))
        for steps in (whole("e", tokens), tail_one_by_one("e", tokens, tail=3), portions("e", tokens, [2, 61])):
            got = run_steps(runner, steps)
            compare_rows({k: v for k, v in got.items() if k[1] >= n - 3}, {"e": plain}, TOL[dtype])
    assert changed > 0.05  # the mark does show in the last row


def test_first_tokens_of_a_sequence(taborax_folders):
    """Requests of one, two and three tokens, whole and token by token: one key beside the sink,
    the first page half empty."""
    for name in ("mixed", "straight", "awkward"):
        folder, vocab = taborax_folders[name, False], CONFIGS[name]["vocab"]
        reqs = {f"s{n}": random_tokens(n, vocab, 30 + n) for n in (1, 2, 3, 6)}
        plain = plain_rows(folder, reqs)
        runner = runner_for(folder, "float32", tokens=64)
        for rid, toks in reqs.items():
            compare_rows(run_steps(runner, whole(rid, toks)), plain, TOL["float32"])
            compare_rows(run_steps(runner, portions(rid, toks, [1])), plain, TOL["float32"])


def test_the_sink_shows_in_the_first_tokens(tmp_path):
    """The plain model itself: with ordinary softmax in place of the unit sink the first rows
    change, so the tests above do tell a sink that is left out."""
    config = one_layer(attention_layer(2, 1, 16, 0.25, rot={"base": 20.0, "dims": 8}), width=32, vocab=64)
    folder = make_folder(tmp_path / "sink", config, seed=2)
    cfg, w = load_plain(folder)
    tokens = random_tokens(5, 64, 1)
    with_sink = pt.forward(tokens, w, cfg)
    kept = pt.softmax_with_unit_sink
    try:
        pt.softmax_with_unit_sink = lambda s: torch.softmax(s, dim=-1)
        without = pt.forward(tokens, w, cfg)
    finally:
        pt.softmax_with_unit_sink = kept
    assert float((with_sink - without).abs().max()) > 1e-2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(taborax_folders, dtype):
    """A short prompt and 400 tokens decoded one by one through recorded steps."""
    folder, vocab = taborax_folders["mixed", STEADY[dtype]], MIXED["vocab"]
    tokens = random_tokens(420, vocab, 77)
    plain = plain_rows(folder, {"d": tokens})
    runner = runner_for(folder, dtype, tokens=448)
    got = run_steps(runner, tail_one_by_one("d", tokens, tail=400))
    compare_rows(got, plain, TOL[dtype])
    assert all(step.captured for step in runner.recorded.values()) and runner.recorded


@pytest.mark.parametrize("name", ["mixed", "awkward"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(taborax_folders, dtype, name):
    """``Engine.generate``: the scheduler cuts prompts into portions beside decoding requests;
    the tokens are the plain model's greedy tokens (in bfloat16: each token is, for the plain
    logits of its own history, within rounding of the best)."""
    from tokasaurus_amd.config.engine_config import EngineConfig
    from tokasaurus_amd.engine.engine import Engine
    from tokasaurus_amd.sampling import SamplingParams

    folder, vocab = taborax_folders[name, STEADY[dtype]], CONFIGS[name]["vocab"]
    prompts = [random_tokens(n, vocab, 10 + n) for n in (5, 40, 23, 1, 64)]
    engine = Engine(EngineConfig(model=str(folder), dtype=dtype, page_size=PAGE, kv_cache_num_tokens=512, max_seqs_per_forward=3,
                                 max_tokens_per_forward=24, allocator_sanity_checks=True))
    done = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    cfg, w = load_plain(folder)
    for prompt, c in zip(prompts, done):
        assert len(c.tokens) == 12 and c.finish_reason == "length"
        ids = list(prompt)
        for tok in c.tokens:
            logits = pt.forward(ids, w, cfg)[-1]
            if dtype == "float32":
                assert tok == int(logits.argmax()), f"token {tok}, plain {int(logits.argmax())}"
            else:
                assert float(logits.max() - logits[tok]) < 0.05 * float(logits.std()) + 0.05
            ids.append(tok)
    assert engine.runner.manager.requests == {}


def test_command_line_and_trace_replay(taborax_folders, tmp_path):
    """``bin/toka`` generates from a Taborax folder (also from a config.json alone, with random
    weights), and ``bin/trace_run`` replays given tokens step by step: its logits are the plain model's."""
    import os
    import subprocess
    import sys

    import numpy as np

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, vocab = taborax_folders["straight", False], CONFIGS["straight"]["vocab"]
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
            assert tok == int(pt.forward(ids, w, cfg)[-1].argmax())
            ids.append(tok)
    model = tmp_path / "fresh"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(CONFIGS["awkward"]))
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


def random_config(seed: int) -> dict:
    """A Taborax configuration drawn from lists of sizes that hold the kernels' comfortable values and awkward ones."""
    import random

    rng = random.Random(seed)
    width = rng.choice([48, 64, 72, 96, 136])
    layers = []
    for _ in range(rng.randint(2, 5)):
        kind = rng.choice(["dense", "moe", "moe", None])
        mlp = None
        if kind == "dense":
            mlp = dense(rng.choice([40, 64, 100, 160]))
        elif kind == "moe":
            experts, identity = rng.randint(2, 12), rng.choice([0, 0, 1, 3])
            n_all = experts + identity
            count = rng.choice([g for g in (1, 2, 3, 4, 5) if n_all % g == 0])
            keep = rng.randint(1, count)
            top = rng.randint(1, min(4, n_all // count * keep))
            mlp = moe(rng.choice([8, 20, 32, 48]), experts, top, identity=identity if identity else None,
                      groups=(count, keep) if rng.random() < 0.8 or count > 1 else None, shared=rng.choice([None, 16, 40]))
        if rng.random() < 0.5:
            layers.append(latent_layer(rng.choice([1, 2, 3, 4, 6, 8]), rng.choice([8, 16, 24, 32, 40, 64]), rng.choice([8, 16, 32, 48, 64]),
                                       rng.choice([8, 12, 24, 40]), rng.choice([8, 16, 24, 48, 64, 80, 128]), rng.uniform(0.05, 0.4), mlp))
        else:
            kv, dim = rng.choice([1, 2, 4]), rng.choice([8, 16, 32, 64, 128])
            rot = None if rng.random() < 0.25 else {"base": rng.choice([10.0, 1000.0, 1e6]), "dims": 2 * rng.randint(1, dim // 2)}
            layers.append(attention_layer(kv * rng.choice([1, 2, 3, 4]), kv, dim, rng.uniform(0.05, 0.4), rot=rot, mlp=mlp))
    cfg = {"architecture": "Taborax", "vocab": rng.randint(50, 300), "width": width, "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])},
           "layers": layers}
    if rng.random() < 0.7:
        start = rng.randint(0, len(layers) - 1)
        cfg["loop"] = {"start": start, "stop": rng.randint(start + 1, len(layers)), "times": rng.randint(1, 3)}
    return cfg


@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(tmp_path, seed):
    """Drawn configurations in 32-bit: a prompt whole, its tail token by token, in portions, and beside another request."""
    config = random_config(seed)
    folder = make_folder(tmp_path / "m", config, seed=seed)
    reqs = {"a": random_tokens(75, config["vocab"], seed), "b": random_tokens(22, config["vocab"], seed + 100)}
    plain = plain_rows(folder, reqs)
    runner = runner_for(folder, "float32", tokens=192)
    tol = TOL["float32"]
    compare_rows(run_steps(runner, whole("a", reqs["a"])), plain, tol)
    compare_rows(run_steps(runner, tail_one_by_one("a", reqs["a"], tail=20)), plain, tol)
    compare_rows(run_steps(runner, portions("a", reqs["a"], [2, 17, 1, 33, 3])), plain, tol)
    compare_rows(run_steps(runner, mixed_trace(reqs, seed, max_live=2)), plain, tol)
    assert runner.manager.requests == {}
