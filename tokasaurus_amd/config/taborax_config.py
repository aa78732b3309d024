"""The configuration of a Taborax model, read from its ``config.json``.

The file lists the layers one by one; every size and every constant that may differ between
two models of the design is taken from it.  Keys:

    architecture: "Taborax"       vocab, width                norm.eps
    loop: absent or null | {start, stop, times}   layers start .. stop-1 run ``times`` times in a row
    layers[i].type: "latent_attention" | "attention"
    layers[i].mlp: null | {"kind": "dense", "ff": n}
                        | {"kind": "moe", "expert": {ff}, "router": {experts, top, identity, groups: {count, keep}},
                           "shared": absent or null | {ff}}
    latent_attention mixer: heads, dim, vdim, q_rank, kv_rank, scale
    attention mixer:        heads, kv_heads, dim, vdim, scale, rot: absent or null | {base, dims}
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from tokasaurus_amd.config.kupuzen_config import _need
from tokasaurus_amd.config.model_config import ConfigError


@dataclass(frozen=True)
class LatentAttentionLayer:
    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float


@dataclass(frozen=True)
class SharedKeyAttentionLayer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float | None  # None: no rotation
    rot_dims: int


@dataclass(frozen=True)
class DenseFF:
    ff: int


@dataclass(frozen=True)
class ExpertsFF:
    ff: int  # inner size of a routed expert
    experts: int
    top: int
    identity: int
    groups: int
    keep: int
    shared_ff: int | None  # inner size of the expert every token uses, None for none


@dataclass(frozen=True)
class TaboraxLayer:
    kind: str
    mixer: LatentAttentionLayer | SharedKeyAttentionLayer
    ff: DenseFF | ExpertsFF | None


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class TaboraxConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: tuple[TaboraxLayer, ...]
    loop: Loop | None = None
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "TaboraxConfig":
        layers = []
        for i, layer in enumerate(_need(d, "layers", "the file")):
            where = f"layers[{i}]"
            kind = _need(layer, "type", where)
            m = _need(layer, "mixer", where)
            mw = f"{where}.mixer"
            if kind == "latent_attention":
                mixer: LatentAttentionLayer | SharedKeyAttentionLayer = LatentAttentionLayer(
                    heads=int(_need(m, "heads", mw)), dim=int(_need(m, "dim", mw)), vdim=int(_need(m, "vdim", mw)),
                    q_rank=int(_need(m, "q_rank", mw)), kv_rank=int(_need(m, "kv_rank", mw)), scale=float(_need(m, "scale", mw)))
            elif kind == "attention":
                rot = m.get("rot")
                mixer = SharedKeyAttentionLayer(
                    heads=int(_need(m, "heads", mw)), kv_heads=int(_need(m, "kv_heads", mw)), dim=int(_need(m, "dim", mw)),
                    vdim=int(_need(m, "vdim", mw)), scale=float(_need(m, "scale", mw)),
                    rot_base=float(_need(rot, "base", f"{mw}.rot")) if rot else None,
                    rot_dims=int(_need(rot, "dims", f"{mw}.rot")) if rot else 0)
            else:
                raise ConfigError(f"config.json: {where} has type {kind!r}; known: latent_attention, attention")
            mlp = layer.get("mlp")
            ff: DenseFF | ExpertsFF | None = None
            if mlp is not None:
                fw = f"{where}.mlp"
                if mlp.get("kind") == "dense":
                    ff = DenseFF(int(_need(mlp, "ff", fw)))
                elif mlp.get("kind") == "moe":
                    r = _need(mlp, "router", fw)
                    g = r.get("groups") or {}
                    shared = mlp.get("shared")
                    ff = ExpertsFF(
                        ff=int(_need(_need(mlp, "expert", fw), "ff", f"{fw}.expert")),
                        experts=int(_need(r, "experts", f"{fw}.router")), top=int(_need(r, "top", f"{fw}.router")),
                        identity=int(r.get("identity") or 0),
                        groups=int(g.get("count") or 1), keep=int(g.get("keep") or g.get("count") or 1),
                        shared_ff=int(_need(shared, "ff", f"{fw}.shared")) if shared else None)
                else:
                    raise ConfigError(f"config.json: {fw} has kind {mlp.get('kind')!r}; known: dense, moe")
            layers.append(TaboraxLayer(kind, mixer, ff))
        loop = d.get("loop")
        eos = d.get("eos_token_id")
        cfg = cls(
            vocab=int(_need(d, "vocab", "the file")),
            width=int(_need(d, "width", "the file")),
            norm_eps=float(_need(_need(d, "norm", "the file"), "eps", "norm")),
            layers=tuple(layers),
            loop=Loop(int(_need(loop, "start", "loop")), int(_need(loop, "stop", "loop")), int(_need(loop, "times", "loop"))) if loop else None,
            eos_token_ids=() if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos)),
        )
        cfg.validate()
        return cfg

    def run_order(self) -> list[tuple[int, bool]]:
        """(layer, whether a pass of the loop begins with it) in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        a, b = self.loop.start, self.loop.stop
        order = [(i, False) for i in range(a)]
        for _ in range(self.loop.times):
            order += [(i, i == a) for i in range(a, b)]
        return order + [(i, False) for i in range(b, n)]

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            raise ConfigError("config.json: vocab, width and the number of layers must be positive")
        if self.loop is not None and not (0 <= self.loop.start < self.loop.stop <= len(self.layers) and self.loop.times >= 1):
            raise ConfigError(f"config.json: loop {self.loop} names no run of the {len(self.layers)} layers")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if isinstance(m, LatentAttentionLayer):
                if min(m.heads, m.dim, m.vdim, m.q_rank, m.kv_rank) <= 0:
                    raise ConfigError(f"config.json: layers[{i}]: sizes of the latent attention must be positive")
            else:
                if min(m.heads, m.kv_heads, m.dim, m.vdim) <= 0 or m.heads % m.kv_heads:
                    raise ConfigError(f"config.json: layers[{i}]: {m.heads} heads over {m.kv_heads} kv heads of sizes {m.dim}, {m.vdim}")
                if m.vdim != m.dim:
                    raise ConfigError(f"config.json: layers[{i}]: the values are the keys, so vdim {m.vdim} must be dim {m.dim}")
                if m.rot_base is not None and (m.rot_dims % 2 or not 0 < m.rot_dims <= m.dim):
                    raise ConfigError(f"config.json: layers[{i}] rotates {m.rot_dims} of {m.dim} elements")
            f = layer.ff
            if isinstance(f, ExpertsFF):
                n_all = f.experts + f.identity
                if min(f.ff, f.experts, f.top, f.groups, f.keep) <= 0 or f.identity < 0:
                    raise ConfigError(f"config.json: layers[{i}].mlp: sizes of the mixture must be positive")
                if n_all % f.groups or f.keep > f.groups or f.top > (n_all // f.groups) * f.keep:
                    raise ConfigError(f"config.json: layers[{i}].mlp: {n_all} experts in {f.groups} groups of which {f.keep} stay "
                                      f"open cannot give {f.top} choices")
            elif isinstance(f, DenseFF) and f.ff <= 0:
                raise ConfigError(f"config.json: layers[{i}].mlp.ff must be positive")
