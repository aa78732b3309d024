"""Kupuzen as a choice of parts: a scaled embedding into a 32-bit residual stream; blocks whose
mixer and feed-forward run side by side on two norms of the same stream, scaled by one
multiplier; per layer either grouped-query attention (whole-projection norms, rotation of
neighbouring elements, sliding window, sinks, optionally another layer's keys and values) or
the gated delta rule with a decay per key channel; a soft-capped head.  Checkpoint names:
``embed``, ``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.gate|up|down``, ``final.norm``, ``head``.

The two low ranks of a delta-rule layer come with the configuration when it says them or has
taken them from the checkpoint's shapes (``KupuzenConfig.with_tensor_shapes``); a model made
without either takes ``default_rank``.
"""

from __future__ import annotations

from tokasaurus_amd.config.kupuzen_config import AttentionLayer, KupuzenConfig
from tokasaurus_amd.models.spec import ModelSpec, RunEntry
from tokasaurus_amd.parts.base import PartSpec

MAX_POSITIONS = 1 << 30  # the rotation computes its angles from the position: no table ends them


def default_rank(width: int) -> int:
    """The low rank of a delta-rule layer's decay and gate projections when no checkpoint says."""
    return max(8, (width // 16 + 7) // 8 * 8)


def kupuzen_spec(cfg: KupuzenConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("stream_rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "name": name, "unit_offset": True})

    # a layer whose keys another layer reads keeps them as far back as its furthest reader looks
    keep = {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if isinstance(m, AttentionLayer):
            owner = i if m.kv_from is None else m.kv_from
            seen = keep.get(owner, m.window)
            keep[owner] = 0 if (seen == 0 or m.window == 0) else max(seen, m.window)

    layers, order = [], []
    for i, layer in enumerate(cfg.layers):
        m, p = layer.mixer, f"l{i}.mix"
        if isinstance(m, AttentionLayer):
            position = None
            if m.rotary is not None:
                position = PartSpec("rotary_interleaved", {"dims": m.rotary.dims, "base": m.rotary.base,
                                                           "scaling": m.rotary.scaling_dict()})
            own = m.kv_from is None
            mixer = PartSpec("grouped_attention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
                "value_dim": m.vdim, "scale": m.scale, "position": position, "window": m.window,
                "cache_window": keep[i if own else m.kv_from],
                "projection_norm": {"q": f"{p}.q.norm", "k": f"{p}.k.norm", "eps": cfg.norm_eps},
                "sink_name": f"{p}.sink", "own_kv": own,
                "names": {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o"},
            })
            order.append(RunEntry(i, cache_of=m.kv_from))
        else:
            mixer = PartSpec("channel_delta_rule", {
                "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
                "value_dim": m.vdim, "taps": m.taps, "decay_rank": m.decay_rank or default_rank(cfg.width),
                "gate_rank": m.gate_rank or default_rank(cfg.width),
                "norm_eps": cfg.norm_eps,
                "names": {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "q_conv": f"{p}.q.conv", "k_conv": f"{p}.k.conv",
                          "v_conv": f"{p}.v.conv", "b": f"{p}.b", "a1": f"{p}.a1", "a2": f"{p}.a2", "g1": f"{p}.g1",
                          "g2": f"{p}.g2", "o": f"{p}.o", "A_log": f"{p}.A_log", "dt_bias": f"{p}.dt_bias", "norm": f"{p}.norm"},
            })
            order.append(RunEntry(i))
        params = {"mixer_norm": norm(f"l{i}.norm1"), "mixer": mixer, "residual_mult": cfg.residual_mult}
        if layer.ff is not None:
            params["ff_norm"] = norm(f"l{i}.norm2")
            params["feed_forward"] = PartSpec("swiglu", {
                "hidden_size": cfg.width, "intermediate_size": layer.ff,
                "names": {"gate": f"l{i}.mlp.gate", "up": f"l{i}.mlp.up", "down": f"l{i}.mlp.down"}})
        layers.append(PartSpec("parallel_residual", params))
    return ModelSpec(
        vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "embed",
                                               "scale": cfg.embedding_scale, "stream_f32": True}),
        head=PartSpec("norm_linear", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "head",
                                      "norm": norm("final.norm"), "softcap": cfg.logit_softcap}),
        layers=tuple(layers),
        run_order=tuple(order),
        max_positions=MAX_POSITIONS,
        eos_token_ids=cfg.eos_token_ids,
    )
