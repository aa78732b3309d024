"""Attention whose keys and values are expanded, head by head, from one small latent a token, and
only that latent is cached.

Per token: the query latent ``cq = norm(W_dq h)`` and the key/value latent ``c = norm(W_dkv h)``
(RMS norms with weights, 32-bit); ``q = W_uq cq``; per head ``k = W_uk c`` and ``v = W_uv c``;
``score = (q . k) * scale`` over every earlier token and the token itself, an ordinary softmax,
no positions; the output projection reads the heads side by side.

Two forms of the same sums, chosen request by request in every step:

* **Single tokens** never expand a cached token's keys or values.  Since ``q_h . (W_uk,h c) =
  (W_uk,h^T q_h) . c`` and ``sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j``, a head's query is taken
  into the latent's space (a matrix a head, ``ops.head_linear``), the attention runs with ONE
  key/value head whose keys and values are both the latent (every query head reads it: the
  arithmetic intensity of the cache is that of ``num_heads`` queries a key), and the head's
  result is taken from the latent's space to its values by ``W_uv,h``.
* **Portions of prompts** expand: in the latent's space a score costs ``kv_rank`` multiply-adds
  a head instead of ``key_dim``, which for many queries outweighs expanding every key once.  The
  latents of the portion's requests are read back from the pages (``ops.gather_keys``), one
  product gives all heads' keys and values, and they go into pages of the step's own (a block
  table that counts up) over which the ordinary attention runs.  Nothing of it is kept.

The pages hold the latent twice, once in the key layout and once in the value layout,
``2 * kv_rank`` numbers a token and layer where expanded keys and values would take
``num_heads * (key_dim + value_dim)``.

Scores, softmax weights and norms are 32-bit arithmetic in either storage type; the kernels are
those of ``grouped_attention`` (``ops.qk_prepare`` norms both latents and appends,
``ops.attention_tile_f32`` or, for sizes it does not take, ``ops.paged_attention_generic``).
"""

from __future__ import annotations

import numpy as np
import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.kernels.upload import upload
from tokasaurus_amd.parts.base import MATRIX, MIXERS, NORM_WEIGHT, CacheNeed, CacheView, Mixer, StepContext, TensorSpec
from tokasaurus_amd.parts.grouped_attention import tile_plan
from tokasaurus_amd.parts.linear import Linear, Placer


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, q_rank: int, kv_rank: int, scale: float,
                 norm_eps: float, names: dict[str, str], key_chunk: int = 256):
        """``names``: checkpoint names under the keys dq, dkv ([rank, hidden]), dq_norm, dkv_norm
        ([rank]), uq ([heads * key_dim, q_rank]), uk ([heads * key_dim, kv_rank]), uv
        ([heads * value_dim, kv_rank]), o ([hidden, heads * value_dim]).  ``key_chunk``: in steps of
        few tokens a request's keys are cut at multiples of this many among workgroups (0: never)."""
        self.key_chunk = int(key_chunk)
        self.heads_a_call = num_heads  # query heads one call of the plain attention kernel takes (set when the cache is checked)
        self.hidden_size, self.num_heads = hidden_size, num_heads
        self.key_dim, self.value_dim, self.q_rank, self.kv_rank = int(key_dim), int(value_dim), int(q_rank), int(kv_rank)
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.names = dict(names)
        self.down = Linear(hidden_size, [names["dq"], names["dkv"]], [self.q_rank, self.kv_rank])
        self.up_q = Linear(self.q_rank, [names["uq"]], [num_heads * self.key_dim])
        self.out = Linear(num_heads * self.value_dim, [names["o"]], [hidden_size])
        # all heads' keys and values of a latent in one product (prompt portions)
        self.expand = Linear(self.kv_rank, [names["uk"], names["uv"]], [num_heads * self.key_dim, num_heads * self.value_dim])
        self.q_norm_weight = self.c_norm_weight = None
        self.to_latent: torch.Tensor | None = None  # [heads, kv_rank, key_dim]: W_uk,h transposed
        self.from_latent: torch.Tensor | None = None  # [heads, value_dim, kv_rank]: W_uv,h

    def tensor_specs(self) -> list[TensorSpec]:
        n, H = self.names, self.num_heads
        return self.down.tensor_specs() + self.up_q.tensor_specs() + self.out.tensor_specs() + self.expand.tensor_specs() + [
            TensorSpec(n["dq_norm"], (self.q_rank,), NORM_WEIGHT),
            TensorSpec(n["dkv_norm"], (self.kv_rank,), NORM_WEIGHT),
        ]

    def cache_need(self) -> CacheNeed:
        return CacheNeed(1, self.kv_rank, 0, 0)

    def check_cache(self, page_size: int, dtype: torch.dtype) -> None:
        if ops.attention_tile_f32_fits(self.num_heads, 1, self.kv_rank, self.kv_rank, page_size):
            ops.key_pages_shape(1, 1, page_size, self.kv_rank, padded=True)
            ops.value_pages_shape(1, 1, page_size, self.kv_rank)
        else:
            # the plain kernel bounds the heads that share a kv head (their number times the latent's size):
            # more heads than it takes at once go in several calls
            ops.key_pages_shape(1, 1, page_size, self.kv_rank, padded=True)
            ops.value_pages_shape(1, 1, page_size, self.kv_rank)
            m = self.num_heads
            while m > 1 and not ops.paged_attention_generic_fits(m, 1, self.kv_rank, self.kv_rank):
                m = (m + 1) // 2
            ops.check_attention_shape(dtype, m, 1, self.kv_rank, page_size, value_dim=self.kv_rank, generic_only=True)
            self.heads_a_call = m

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        for lin in (self.down, self.up_q, self.out, self.expand):
            lin.load(tensors, placer)
        n, H = self.names, self.num_heads

        def f32(name: str) -> torch.Tensor:
            return placer.place(("vector_f32", name), lambda: tensors[name].to(torch.float32).contiguous().to(placer.device))

        self.q_norm_weight, self.c_norm_weight = f32(n["dq_norm"]), f32(n["dkv_norm"])
        self.to_latent = placer.place(("heads_transposed", n["uk"]), lambda: tensors[n["uk"]].to(placer.dtype).view(
            H, self.key_dim, self.kv_rank).transpose(1, 2).contiguous().to(placer.device))
        self.from_latent = placer.place(("heads", n["uv"]), lambda: tensors[n["uv"]].to(placer.dtype).view(
            H, self.value_dim, self.kv_rank).contiguous().to(placer.device))

    def _attend(self, h: torch.Tensor, ctx: StepContext, cache: CacheView, rows: torch.Tensor | None) -> torch.Tensor:
        assert cache is not None and cache.writable, "latent attention keeps its latent in a cache of its own"
        H, r = self.num_heads, self.kv_rank
        lat = self.down(h)  # [cq | c]
        # both latents normed (each over its whole length), the key/value latent appended as key and as value
        ops.qk_prepare(lat, ctx.positions, ctx.token_req, cache.block_table, self.q_norm_weight, self.c_norm_weight,
                       self.norm_eps, None, cache.keys, cache.values, 1, 1, r, r, cache.page_size,
                       query_dim=self.q_rank, values_are_keys=True)
        cq = lat[:, : self.q_rank]
        if lat.dtype != torch.float32 and (self.q_rank % 8 or lat.stride(0) % 8):
            cq = torch.empty((lat.shape[0], self.q_rank), dtype=lat.dtype, device=lat.device).copy_(cq)
        q = self.up_q(cq)  # [tokens, heads * key_dim]
        # the requests that bring portions come first in a step; their tokens are the step's first rows
        portions = int(ctx.extras.get("num_portions", 0))
        first_single = ctx.host_q_start[portions] if portions else 0
        if portions and ops.attention_tile_f32_fits(H, H, self.key_dim, self.value_dim, cache.page_size):
            o = self._over_expanded(q, ctx, cache, portions)
            if first_single < ctx.num_tokens:
                o[first_single:] = self._over_latent(q[first_single:], ctx, cache, first_single, ctx.num_requests - portions)
        else:
            o = self._over_latent(q, ctx, cache, 0, None)
        return o if rows is None else ops.gather_rows(o, rows)

    def _over_latent(self, q: torch.Tensor, ctx: StepContext, cache: CacheView, first_row: int, last_requests: int | None) -> torch.Tensor:
        """Attention in the latent's space for the step's rows from ``first_row`` on (``q`` holds those
        rows), which belong to the step's last ``last_requests`` requests, one token each (None: all
        rows of all requests)."""
        H, r = self.num_heads, self.kv_rank
        ql = ops.head_linear(q, self.to_latent)  # [rows, heads * kv_rank]
        if ops.attention_tile_f32_fits(H, 1, r, r, cache.page_size):
            gg = ops.attention_tile_heads(H, ctx.max_q_len if last_requests is None else 1)
            tile_req, tile_row0 = tile_plan(ctx, 16 // gg)
            if last_requests is not None:  # a request of one token is one tile, whatever a tile holds
                tile_req, tile_row0 = tile_req[tile_req.numel() - last_requests:], tile_row0[tile_row0.numel() - last_requests:]
            o = ops.attention_tile_f32(ql, cache.keys, cache.values, cache.block_table, ctx.q_start, ctx.kv_len,
                                       tile_req, tile_row0, H, 1, r, r, cache.page_size, gg, scale=self.scale,
                                       key_chunk=self.key_chunk, longest=ctx.extras.get("kv_bound", ctx.max_kv_len),
                                       first_row=first_row)
        else:
            o = torch.empty((ql.shape[0], H * r), dtype=ql.dtype, device=ql.device)
            for h0 in range(0, H, self.heads_a_call):
                n = min(self.heads_a_call, H - h0)
                part = ops.paged_attention_generic(ql[:, h0 * r :], cache.keys, cache.values, cache.block_table,
                                                   ctx.token_req[first_row:], ctx.positions[first_row:], n, 1, r, cache.page_size,
                                                   scale=self.scale, value_dim=r)
                if n == H:
                    o = part
                else:
                    o[:, h0 * r : (h0 + n) * r] = part
        return ops.head_linear(o, self.from_latent)  # [rows, heads * value_dim]

    def _over_expanded(self, q: torch.Tensor, ctx: StepContext, cache: CacheView, portions: int) -> torch.Tensor:
        """Attention over expanded keys and values for the tokens of the step's first ``portions``
        requests; returns rows for all of the step's tokens, of which only those are written."""
        H, dk, dv, P = self.num_heads, self.key_dim, self.value_dim, cache.page_size
        plan = ctx.extras.get(("expanded_keys_plan", portions, P))
        if plan is None:  # made once a step, shared by the layers
            lens = np.asarray(ctx.host_kv_len[:portions], dtype=np.int64)
            pages = -(-lens // P)
            first_page = np.concatenate([[0], np.cumsum(pages)])
            total = int(lens.sum())
            req = np.repeat(np.arange(portions, dtype=np.int32), lens)
            pos = (np.arange(total, dtype=np.int64) - np.repeat(np.concatenate([[0], np.cumsum(lens)[:-1]]), lens)).astype(np.int32)
            table = np.zeros((portions, int(pages.max())), dtype=np.int32)
            for i in range(portions):
                table[i, : pages[i]] = first_page[i] + np.arange(pages[i])
            dev = upload(np.concatenate([req, pos, table.reshape(-1)]), torch.int32, q.device)
            n_tiles = sum(-(-(ctx.host_q_start[i + 1] - ctx.host_q_start[i]) // 16) for i in range(portions))
            plan = ctx.extras[("expanded_keys_plan", portions, P)] = (
                dev[:total], dev[total : 2 * total], dev[2 * total :].view(portions, -1), int(first_page[-1]), n_tiles)
        req_d, pos_d, table_d, n_pages, n_tiles = plan
        latents = ops.gather_keys(cache.keys, cache.block_table, req_d, pos_d, self.kv_rank, P)
        kv = self.expand(latents)  # [all keys of these requests, heads * key_dim | heads * value_dim]
        # (zeros: the rest of a request's last page is read, with weight zero, and must hold numbers)
        keys = torch.zeros(ops.key_pages_shape(n_pages, H, P, dk, padded=True), dtype=q.dtype, device=q.device)
        values = torch.zeros(ops.value_pages_shape(n_pages, H, P, dv), dtype=q.dtype, device=q.device)
        ops.qk_prepare(kv, pos_d, req_d, table_d, None, None, 0.0, None, keys, values, 0, H, dk, dv, P)
        tile_req, tile_row0 = tile_plan(ctx, 16)
        return ops.attention_tile_f32(q, keys, values, table_d, ctx.q_start, ctx.kv_len, tile_req[:n_tiles], tile_row0[:n_tiles],
                                      H, H, dk, dv, P, 1, scale=self.scale)

    def mix(self, h, ctx, cache, state, rows, out_f32: bool = False):
        return self.out(self._attend(h, ctx, cache, rows), out_f32=out_f32)

    def forward(self, h, residual, ctx, cache, state, rows):
        return self.out(self._attend(h, ctx, cache, rows), residual=residual)
