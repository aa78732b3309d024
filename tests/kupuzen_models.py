"""Small Kupuzen configurations of the tests' own, their model folders, and the plain model's
rows for them.  The configurations differ from one another in every size and option: heads
and their grouping (also in the delta-rule layers), key and value sizes that differ and are
no powers of two (one key size is no multiple of 8), windows from 1 key to none, a layer that
reads another's keys through a wider window than the owner's own, rotated parts from a few
elements to the whole head, with and without wavelength scaling, convolutions of 1 to 5 taps,
layers without a feed-forward, low ranks that are no multiples of 8, no soft cap.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open
from safetensors.torch import save_file

import plain_kupuzen
from tokasaurus_amd.weights import write_random_model


def attention_layer(heads, kv_heads, dim, vdim, scale, window=None, rot=None, kv_from=None, ff=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        mixer["mask"] = {"size": window}
    if rot is not None:
        mixer["rot"] = rot
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def delta_layer(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank, ff=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
             "decay_rank": decay_rank, "gate_rank": gate_rank}
    return {"type": "channel_delta", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


ROT_SCALED = {"base": 10000.0, "dims": 8, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 32}}
ROT_WHOLE = {"base": 300.0, "dims": 24}

# every mechanism in one model; layer 2 reads layer 0's keys through a wider window than layer 0's own
MIXED = {
    "architecture": "Kupuzen", "vocab": 160, "width": 96, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5},
    "residual_mult": 0.5, "logit_softcap": 8.0,
    "layers": [
        attention_layer(6, 3, 24, 16, 0.3, window=9, rot=ROT_SCALED, ff=144),
        delta_layer(4, 2, 24, 40, 3, 12, 20),
        attention_layer(6, 3, 24, 16, 0.25, window=21, rot=ROT_SCALED, kv_from=0, ff=100),
        delta_layer(2, 2, 40, 8, 5, 16, 8, ff=64),
        attention_layer(2, 2, 24, 24, 0.2, rot=ROT_WHOLE, ff=64),
    ],
}
# only delta-rule layers: no cache group at all; one tap (no tail), one head, no soft cap
RECURRENT = {
    "architecture": "Kupuzen", "vocab": 97, "width": 64, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
    "residual_mult": 1.0,
    "layers": [delta_layer(1, 1, 72, 24, 1, 8, 8, ff=96), delta_layer(6, 2, 16, 16, 2, 24, 16)],
}
# only attention: key sizes that are no multiples of 8 (one of them odd), a window of one key, no grouping, no rotation in one layer
WINDOWS = {
    "architecture": "Kupuzen", "vocab": 200, "width": 80, "embedding": {"scale": 0.7}, "norm": {"eps": 1e-4},
    "residual_mult": 0.8, "logit_softcap": 50.0,
    "layers": [
        attention_layer(4, 4, 20, 12, 0.4, window=1, rot={"base": 50.0, "dims": 20}, ff=48),
        attention_layer(3, 1, 7, 5, 0.6, window=11, rot={"base": 30.0, "dims": 6}),
        attention_layer(8, 2, 16, 32, 0.5, window=16, rot={"base": 1000.0, "dims": 4}),
        attention_layer(8, 2, 16, 32, 0.35, window=5, kv_from=2, ff=48),
        attention_layer(2, 1, 32, 8, 0.2, window=64, ff=32),
    ],
}
# sizes that fit nothing: a width, feed-forward sizes, a vocabulary and low ranks that are no multiples of 8 (or of 2),
# delta-rule heads of 48 x 20 and 136 x 12 with grouping, 6 taps, large attention heads without grouping, two
# layers that read one owner's keys, a rotation of the whole head with scaling
AWKWARD = {
    "architecture": "Kupuzen", "vocab": 131, "width": 100, "embedding": {"scale": 1.5}, "norm": {"eps": 1e-6},
    "residual_mult": 0.4, "logit_softcap": 12.0,
    "layers": [
        delta_layer(3, 1, 48, 20, 6, 10, 7, ff=75),
        attention_layer(2, 2, 128, 128, 0.09, window=50, rot={"base": 5000.0, "dims": 128, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 16}}, ff=52),
        attention_layer(2, 2, 128, 128, 0.1, window=70, rot={"base": 5000.0, "dims": 128, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 16}}, kv_from=1),
        delta_layer(2, 1, 136, 12, 2, 5, 9),
        attention_layer(2, 2, 128, 128, 0.08, window=3, rot={"base": 5000.0, "dims": 128, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 16}}, kv_from=1, ff=33),
    ],
}
CONFIGS = {"mixed": MIXED, "recurrent": RECURRENT, "windows": WINDOWS, "awkward": AWKWARD}


def make_folder(folder: Path, config: dict, seed: int, edits: dict | None = None) -> Path:
    """Random weights with the parts scaled so that each mechanism matters to the logits:
    projections of order one a row, peaked attention, decays near one (a long memory), sinks
    of the scores' own size.  ``edits``: name suffix -> function of the tensor, applied last."""
    write_random_model(folder, config, seed)
    path = folder / "model.safetensors"
    tensors = {}
    with safe_open(str(path), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name).float()
            if t.dim() == 2 and not name.endswith(".conv"):
                t = t * (1.0 / (0.02 * t.shape[1] ** 0.5))  # N(0, 1/in): outputs of order one
            if name.endswith(".dt_bias"):
                t = t - 3.0  # softplus near 0.05: a decay of about 0.95 a token
            if name.endswith(".q.norm") or name.endswith(".k.norm"):
                t = t * 1.5
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
    return {rid: plain_kupuzen.forward(config, w, toks).float() for rid, toks in requests.items()}


def compare_rows(got: dict, plain: dict[str, torch.Tensor], tol: float) -> float:
    """Every collected row against the plain row: the root mean square of the difference over
    the vocabulary, relative to that of the plain row.  Names the first wrong (request, position)."""
    worst = 0.0
    for (rid, pos), row in sorted(got.items()):
        ref = plain[rid][pos]
        err = float((row - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-9))
        assert err <= tol, f"request {rid} position {pos}: relative error {err:.3e} (allowed {tol:.1e})"
        worst = max(worst, err)
    return worst


# relative error of a row of logits: summation order in 32-bit; roundings to 8 bits of mantissa in bfloat16
TOL = {"float32": 3e-4, "bfloat16": 6e-2}
