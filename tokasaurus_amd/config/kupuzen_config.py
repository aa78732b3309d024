"""The configuration of a Kupuzen model, read from its ``config.json``.

The file lists the layers one by one; every size and every constant that may differ between
two models of the design is taken from it (or, for the low ranks of a delta-rule layer, from
the shapes of the checkpoint's tensors, which the file does not repeat).  Keys:

    architecture: "Kupuzen"       vocab, width                embedding.scale
    norm.eps                      residual_mult               logit_softcap (absent or null: none)
    layers[i].type: "attention" | "channel_delta"
    layers[i].mlp: null | {"kind": "dense", "ff": n}
    attention mixer:     heads, kv_heads, dim, vdim, scale, mask.size, rot.{base, dims, scaling.{factor, low,
                         high, original}}, kv_from (the layer whose keys and values it reads)
    channel_delta mixer: heads, kv_heads, dim, vdim, conv; optionally decay_rank, gate_rank (the inner sizes
                         of the decay's and the gate's two projections), else taken from the checkpoint's shapes
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from tokasaurus_amd.config.model_config import ConfigError


def _need(d: dict[str, Any], key: str, where: str):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError(f"config.json: {where} lacks {key!r}")
    return d[key]


@dataclass(frozen=True)
class RotaryConfig:
    base: float
    dims: int
    scaling: tuple[tuple[str, float], ...] | None  # factor, low, high, original

    def scaling_dict(self) -> dict[str, float] | None:
        return dict(self.scaling) if self.scaling else None


@dataclass(frozen=True)
class AttentionLayer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int  # 0: every earlier position is seen
    rotary: RotaryConfig | None
    kv_from: int | None


@dataclass(frozen=True)
class DeltaLayer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    taps: int
    decay_rank: int | None = None  # inner size of the decay's two projections; None: not known yet
    gate_rank: int | None = None  # inner size of the output gate's two projections


@dataclass(frozen=True)
class KupuzenLayer:
    kind: str  # "attention" | "channel_delta"
    mixer: AttentionLayer | DeltaLayer
    ff: int | None  # inner size of the dense feed-forward, None for a layer without one


@dataclass(frozen=True)
class KupuzenConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    residual_mult: float
    logit_softcap: float | None
    layers: tuple[KupuzenLayer, ...]
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "KupuzenConfig":
        layers = []
        raw_layers = _need(d, "layers", "the file")
        for i, layer in enumerate(raw_layers):
            where = f"layers[{i}]"
            kind = _need(layer, "type", where)
            m = _need(layer, "mixer", where)
            sizes = {k: int(_need(m, k, f"{where}.mixer")) for k in ("heads", "kv_heads", "dim", "vdim")}
            if kind == "attention":
                rot = m.get("rot")
                rotary = None
                if rot:
                    sc = rot.get("scaling")
                    scaling = None
                    if sc:
                        scaling = tuple((k, float(_need(sc, k, f"{where}.mixer.rot.scaling"))) for k in ("factor", "low", "high", "original"))
                    rotary = RotaryConfig(float(_need(rot, "base", f"{where}.mixer.rot")), int(_need(rot, "dims", f"{where}.mixer.rot")), scaling)
                mask = m.get("mask")
                src = m.get("kv_from")
                mixer: AttentionLayer | DeltaLayer = AttentionLayer(
                    **sizes, scale=float(_need(m, "scale", f"{where}.mixer")),
                    window=int(mask["size"]) if mask and mask.get("size") else 0, rotary=rotary,
                    kv_from=None if src is None else int(src))
            elif kind == "channel_delta":
                mixer = DeltaLayer(**sizes, taps=int(_need(m, "conv", f"{where}.mixer")),
                                   decay_rank=int(m["decay_rank"]) if m.get("decay_rank") else None,
                                   gate_rank=int(m["gate_rank"]) if m.get("gate_rank") else None)
            else:
                raise ConfigError(f"config.json: {where} has type {kind!r}; known: attention, channel_delta")
            mlp = layer.get("mlp")
            ff = None
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp has kind {mlp.get('kind')!r}; known: dense")
                ff = int(_need(mlp, "ff", f"{where}.mlp"))
            layers.append(KupuzenLayer(kind, mixer, ff))
        eos = d.get("eos_token_id")
        cap = d.get("logit_softcap")
        cfg = cls(
            vocab=int(_need(d, "vocab", "the file")),
            width=int(_need(d, "width", "the file")),
            embedding_scale=float(_need(_need(d, "embedding", "the file"), "scale", "embedding")),
            norm_eps=float(_need(_need(d, "norm", "the file"), "eps", "norm")),
            residual_mult=float(_need(d, "residual_mult", "the file")),
            logit_softcap=float(cap) if cap else None,
            layers=tuple(layers),
            eos_token_ids=() if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos)),
        )
        cfg.validate()
        return cfg

    def with_tensor_shapes(self, shapes: dict[str, tuple[int, ...]]) -> "KupuzenConfig":
        """The sizes that only the checkpoint knows, from the shapes of its tensors: the inner
        sizes of a delta-rule layer's low-rank projections (rows of ``l<i>.mix.a1`` and ``.g1``)."""
        from dataclasses import replace

        layers = []
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if isinstance(m, DeltaLayer):
                a1, g1 = shapes.get(f"l{i}.mix.a1"), shapes.get(f"l{i}.mix.g1")
                m = replace(m, decay_rank=int(a1[0]) if a1 else m.decay_rank, gate_rank=int(g1[0]) if g1 else m.gate_rank)
            layers.append(replace(layer, mixer=m))
        return replace(self, layers=tuple(layers))

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("config.json: vocab, width and the number of layers must be positive")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if min(m.heads, m.kv_heads, m.dim, m.vdim) <= 0 or m.heads % m.kv_heads:
                raise ConfigError(f"config.json: layers[{i}]: {m.heads} heads over {m.kv_heads} kv heads of sizes {m.dim}, {m.vdim}")
            if isinstance(m, AttentionLayer):
                if m.rotary and (m.rotary.dims % 2 or not 0 < m.rotary.dims <= m.dim):
                    raise ConfigError(f"config.json: layers[{i}] rotates {m.rotary.dims} of {m.dim} elements")
                if m.kv_from is not None:
                    src = self.layers[m.kv_from].mixer if 0 <= m.kv_from < i else None
                    if not isinstance(src, AttentionLayer) or src.kv_from is not None:
                        raise ConfigError(f"config.json: layers[{i}] reads keys and values of layer {m.kv_from}, "
                                          "which is no earlier attention layer with keys of its own")
                    if (src.kv_heads, src.dim, src.vdim) != (m.kv_heads, m.dim, m.vdim):
                        raise ConfigError(f"config.json: layers[{i}] and layer {m.kv_from}, whose keys it reads, differ in head layout")
            elif m.taps < 1:
                raise ConfigError(f"config.json: layers[{i}] has a convolution of {m.taps} taps")
