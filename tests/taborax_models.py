"""Small Taborax configurations of the tests' own, their model folders, and the plain model's
rows for them.  The configurations differ from one another in every size and option: latent
attention whose key and value sizes differ, latents that are no multiples of 8 or of 16, as large
as the matrix-core kernel takes and larger; grouped attention with one, several and as many kv
heads as heads, a rotation of a few elements, of the whole head, and none; dense feed-forwards,
mixtures with and without identity experts, groups, a shared expert, one choice or several; layers
without a feed-forward; a loop over the first layers, over inner layers, three passes, and none.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open
from safetensors.torch import save_file

import plain_taborax
from tokasaurus_amd.weights import write_random_model


def latent_layer(heads, dim, vdim, q_rank, kv_rank, scale, mlp=None):
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}}


def attention_layer(heads, kv_heads, dim, scale, rot=None, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if rot is not None:
        mixer["rot"] = rot
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, identity=None, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if identity is not None:
        router["identity"] = identity
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


# every mechanism in one model; the inner two layers are passed three times
MIXED = {
    "architecture": "Taborax", "vocab": 160, "width": 96, "norm": {"eps": 1e-5},
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        latent_layer(3, 24, 40, 24, 48, 0.2, dense(144)),
        attention_layer(6, 3, 32, 0.18, rot={"base": 100.0, "dims": 16}, mlp=moe(24, 10, 3, identity=2, groups=(4, 2), shared=40)),
        latent_layer(2, 16, 16, 40, 32, 0.25, moe(32, 5, 1)),
        attention_layer(2, 2, 16, 0.25, rot={"base": 30.0, "dims": 16}),
    ],
}
# no loop; attention without a rotation and with one kv head; a latent that the matrix-core kernel does not take
STRAIGHT = {
    "architecture": "Taborax", "vocab": 97, "width": 80, "norm": {"eps": 1e-6},
    "layers": [
        attention_layer(4, 1, 24, 0.2, mlp=moe(16, 6, 2, identity=0, groups=(3, 3))),
        latent_layer(5, 8, 24, 16, 40, 0.35, dense(56)),
        attention_layer(3, 3, 40, 0.15, rot={"base": 10000.0, "dims": 6}, mlp=dense(120)),
    ],
}
# sizes that fit nothing: a width (no multiple of 4), ranks, expert and feed-forward sizes and a vocabulary that are no multiples of 8
# (or of 2); the loop starts at the first layer; one group of two kept; a single head over an odd latent
AWKWARD = {
    "architecture": "Taborax", "vocab": 131, "width": 90, "norm": {"eps": 1e-4},
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        latent_layer(3, 12, 20, 10, 36, 0.3, moe(20, 9, 2, identity=3, groups=(2, 1), shared=30)),
        attention_layer(5, 1, 28, 0.2, rot={"base": 50.0, "dims": 28}, mlp=dense(75)),
        latent_layer(1, 40, 8, 33, 17, 0.2),
    ],
}
# heads of the sizes of large models: the largest latent the matrix-core kernel takes, heads of 128
LARGE_HEADS = {
    "architecture": "Taborax", "vocab": 120, "width": 128, "norm": {"eps": 1e-5},
    "loop": {"start": 1, "stop": 2, "times": 2},
    "layers": [
        latent_layer(4, 128, 64, 96, 256, 0.09, moe(64, 8, 2, identity=0, groups=(2, 1), shared=64)),
        attention_layer(8, 2, 128, 0.09, rot={"base": 500000.0, "dims": 64}, mlp=dense(256)),
    ],
}
CONFIGS = {"mixed": MIXED, "straight": STRAIGHT, "awkward": AWKWARD, "large_heads": LARGE_HEADS}


def make_folder(folder: Path, config: dict, seed: int, edits: dict | None = None, steady_choice: bool = False) -> Path:
    """Random weights with the parts scaled so that each mechanism matters to the logits:
    projections of order one a row, routers whose scores differ clearly between experts,
    corrections of the scores' own size.  ``edits``: name suffix -> function of the tensor,
    applied last.  ``steady_choice``: the corrections lie 1.5 apart in a shuffled order, so that
    the choice of experts (not their weights) is the same for every token and no comparison in
    bfloat16 rests on which of two nearly equal scores is larger; the 32-bit runs use the
    data-dependent choice."""
    write_random_model(folder, config, seed)
    path = folder / "model.safetensors"
    tensors = {}
    with safe_open(str(path), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name).float()
            if t.dim() == 2:
                t = t * (1.0 / (0.02 * t.shape[1] ** 0.5))  # N(0, 1/in): outputs of order one
            if name.endswith(".router"):
                t = t * 2.0
            if name.endswith(".correction"):
                t = t * 4.0
                if steady_choice:
                    t = 1.5 * torch.argsort(torch.argsort(t)).float() - 0.75 * t.numel()
            for suffix, fn in (edits or {}).items():
                if name.endswith(suffix):
                    t = fn(t)
            tensors[name] = t.to(torch.bfloat16)
    save_file(tensors, str(path))
    return folder


def load_plain(folder: Path, dtype=torch.float64):
    config = json.loads((Path(folder) / "config.json").read_text())
    w = {}
    with safe_open(str(Path(folder) / "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).to(dtype)
    return config, w


def plain_rows(folder: Path, requests: dict[str, list[int]]) -> dict[str, torch.Tensor]:
    config, w = load_plain(folder)
    return {rid: plain_taborax.forward(toks, w, config).float() for rid, toks in requests.items()}


def row_error(row: torch.Tensor, ref: torch.Tensor) -> float:
    return float((row - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-9))


def compare_rows(got: dict, plain: dict[str, torch.Tensor], tol: float, may_flip: float = 0.0) -> float:
    """Every collected row against the plain row: the root mean square of the difference over
    the vocabulary, relative to that of the plain row.  Names the first wrong (request, position).
    ``may_flip``: the share of rows that may miss the bound."""
    worst, over = 0.0, []
    for (rid, pos), row in sorted(got.items()):
        err = row_error(row, plain[rid][pos])
        if err > tol:
            assert may_flip > 0, f"request {rid} position {pos}: relative error {err:.3e} (allowed {tol:.1e})"
            over.append((rid, pos, err))
        worst = max(worst, err)
    assert len(over) <= may_flip * len(got), f"{len(over)} of {len(got)} rows over the bound: {over[:5]}"
    return worst


# relative error of a row of logits: summation order in 32-bit; roundings to 8 bits of mantissa in bfloat16
TOL = {"float32": 3e-4, "bfloat16": 6e-2}
# in bfloat16 a router's choice between two experts of nearly equal score can fall the other way than in the
# plain model: the bfloat16 runs use folders with a steady choice
STEADY = {"float32": False, "bfloat16": True}
