"""Token embedding and the language-model head.

Embedding is a plain row gather without scaling (tokasaurus/model/llama.py:507-518).
The head norms the kept rows and multiplies by the head matrix, which is the
embedding matrix itself when the checkpoint ties them (llama.py:426-467,842-845);
logits leave in 32-bit.
"""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import (EMBEDDINGS, HEADS, MATRIX, NORMS, Embedding, Head, Normed, Part, PartSpec, Prepared,
                                       StepContext, TensorSpec)
from tokasaurus_amd.parts.linear import Linear, Placer


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Embedding):
    def __init__(self, vocab_size: int, hidden_size: int, name: str, scale: float | None = None, stream_f32: bool = False):
        """``scale``: every row is multiplied by it.  ``stream_f32``: the rows leave in 32-bit
        whatever the table's storage type (a model that keeps its residual stream in 32-bit)."""
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.name = name
        self.scale = None if scale is None else float(scale)
        self.stream_f32 = bool(stream_f32)
        if self.scale is not None and not self.stream_f32:
            raise ValueError("a scaled embedding writes a 32-bit stream (stream_f32=True)")
        self.table: torch.Tensor | None = None

    def tensor_specs(self) -> list[TensorSpec]:
        return [TensorSpec(self.name, (self.vocab_size, self.hidden_size), MATRIX)]

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        host = tensors[self.name]
        self.table = placer.place(
            ("row_major", self.name), lambda: host.to(dtype=placer.dtype).contiguous().to(placer.device)
        )

    def forward(self, ctx: StepContext) -> torch.Tensor:
        if self.stream_f32:
            return ops.embed_scaled(ctx.token_ids, self.table, 1.0 if self.scale is None else self.scale, ctx.last_token)
        return ops.embed_gather(ctx.token_ids, self.table, ctx.last_token)


@HEADS.register("norm_linear")
class LMHead(Head):
    def __init__(self, vocab_size: int, hidden_size: int, name: str, norm: PartSpec, softcap: float | None = None):
        """``softcap``: the logits leave as softcap * tanh(logits / softcap)."""
        self.vocab_size = vocab_size
        self.hidden_size = hidden_size
        self.softcap = float(softcap) if softcap else None
        self.norm = NORMS.build(norm)
        self.proj = Linear(hidden_size, [name], [vocab_size])

    def children(self) -> list[Part]:
        return [self.norm]

    def entry_norm(self):
        return self.norm

    def tensor_specs(self) -> list[TensorSpec]:
        return self.norm.tensor_specs() + self.proj.tensor_specs()

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        self.norm.load(tensors, placer)
        self.proj.load(tensors, placer)

    takes_out = True

    def forward(self, x: torch.Tensor, prepared: Prepared | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
        logits = self.proj(Normed(x, self.norm, prepared), out_f32=True, out=out)
        return ops.softcap_(logits, self.softcap) if self.softcap is not None else logits
