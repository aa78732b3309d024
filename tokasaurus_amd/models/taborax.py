"""Taborax as a choice of parts: a plain embedding into a 32-bit residual stream; blocks with a
norm in front of and behind each sublayer; per layer either attention over a cached latent
(keys and values expanded head by head from it, no positions) or grouped-query attention whose
values are its keys, with a rotation of the halves of a head's leading part and a unit sink in
the softmax; per layer a squared-relu feed-forward, a mixture of gated experts with grouped
routing, identity experts and a shared expert, or none; a run of layers that is passed several
times with the same weights, each pass with caches of its own and begun by mixing the
embedding's output back into the stream.  Checkpoint names: ``embed``, ``loop.in``,
``l<i>.norm1|norm1b|norm2|norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from tokasaurus_amd.config.taborax_config import DenseFF, ExpertsFF, LatentAttentionLayer, TaboraxConfig
from tokasaurus_amd.models.spec import ModelSpec, RunEntry
from tokasaurus_amd.parts.base import PartSpec

MAX_POSITIONS = 1 << 30  # the rotation computes its angles from the position: no table ends them


def taborax_spec(cfg: TaboraxConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("stream_rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "name": name})

    layers, unused = [], []
    for i, layer in enumerate(cfg.layers):
        m, p = layer.mixer, f"l{i}.mix"
        if isinstance(m, LatentAttentionLayer):
            mixer = PartSpec("latent_attention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "q_rank": m.q_rank,
                "kv_rank": m.kv_rank, "scale": m.scale, "norm_eps": cfg.norm_eps,
                "names": {"dq": f"{p}.dq", "dq_norm": f"{p}.dq.norm", "uq": f"{p}.uq", "dkv": f"{p}.dkv",
                          "dkv_norm": f"{p}.dkv.norm", "uk": f"{p}.uk", "uv": f"{p}.uv", "o": f"{p}.o"}})
        else:
            position = None
            if m.rot_base is not None:
                position = PartSpec("rotary_halves", {"dims": m.rot_dims, "base": m.rot_base})
            mixer = PartSpec("grouped_attention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
                "value_dim": m.vdim, "scale": m.scale, "position": position, "sink_value": 0.0, "values_are_keys": True, "key_chunk": 256,
                "names": {"q": f"{p}.q", "k": f"{p}.k", "o": f"{p}.o"}})
        params = {"mixer_norm": norm(f"l{i}.norm1"), "mixer": mixer, "mixer_post_norm": norm(f"l{i}.norm1b")}
        f, q = layer.ff, f"l{i}.mlp"
        if f is None:
            unused += [f"l{i}.norm2", f"l{i}.norm2b"]
        else:
            params["ff_norm"], params["ff_post_norm"] = norm(f"l{i}.norm2"), norm(f"l{i}.norm2b")
            if isinstance(f, DenseFF):
                params["feed_forward"] = PartSpec("squared_relu", {
                    "hidden_size": cfg.width, "intermediate_size": f.ff, "names": {"up": f"{q}.up", "down": f"{q}.down"}})
            else:
                assert isinstance(f, ExpertsFF)
                params["feed_forward"] = PartSpec("routed_experts", {
                    "hidden_size": cfg.width, "expert_size": f.ff, "num_experts": f.experts, "top": f.top,
                    "identity": f.identity, "groups": f.groups, "keep": f.keep, "shared_size": f.shared_ff,
                    "names": {"router": f"{q}.router", "correction": f"{q}.correction", "expert": q + ".e{e}",
                              "shared": f"{q}.shared", "shared_gate": f"{q}.shared.sg"}})
        layers.append(PartSpec("sandwich_norm", params))
    connectors = ()
    if cfg.loop is not None:
        connectors = (PartSpec("embedding_mix", {"hidden_size": cfg.width, "name": "loop.in"}),)
    return ModelSpec(
        vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "embed",
                                               "stream_f32": True}),
        head=PartSpec("norm_linear", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "head",
                                      "norm": norm("final.norm")}),
        layers=tuple(layers),
        # a layer that is passed again is named again: every use has a cache of its own
        run_order=tuple(RunEntry(i, before=0 if first else None) for i, first in cfg.run_order()),
        connectors=connectors,
        max_positions=MAX_POSITIONS,
        eos_token_ids=cfg.eos_token_ids,
        # a layer without a feed-forward may still carry the two norms around it
        ignorable_tensors=tuple(unused),
    )
