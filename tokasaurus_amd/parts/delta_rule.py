"""The gated delta rule with one decay per head and key channel: a mixer that keeps, per
request, a matrix per head instead of keys and values.

Per token: q, k (``num_kv_heads`` heads of ``key_dim``) and v (``num_heads`` heads of
``value_dim``) are projections that pass a short causal convolution per channel and silu; q and
k become unit vectors per head (q times key_dim^-1/2); beta = sigmoid(W_b h) per head; the decay
g = exp(-exp(A_log) * softplus(W_a2 W_a1 h + dt_bias)) has one number per head and key channel.
Per head, in this order: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  The
head's o is divided by its root mean square, multiplied by a weight shared by the heads and by
sigmoid(W_g2 W_g1 h), and the output projection follows.

The projections are products in the storage type; what enters the recurrence (unit norms,
beta, decays, the state) and the norm behind it are 32-bit.  The state (the matrices and the
last inputs of the convolutions) is one row of 32-bit numbers in the request's slot, zero when
a request takes the slot; a step of any cut continues from it.
"""

from __future__ import annotations

import torch

from tokasaurus_amd.kernels import ops
from tokasaurus_amd.parts.base import CONV, MATRIX, MIXERS, NORM_WEIGHT, VECTOR, Mixer, StateNeed, StepContext, TensorSpec
from tokasaurus_amd.parts.linear import Linear, Placer


@MIXERS.register("channel_delta_rule")
class ChannelDeltaRule(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, taps: int,
                 decay_rank: int, gate_rank: int, norm_eps: float, names: dict[str, str]):
        """``names``: checkpoint names under the keys q, k, v (matrices), q_conv, k_conv, v_conv
        ([channels, taps], the last column is the current token's), b, a1, a2, g1, g2, o
        (matrices), A_log ([heads]), dt_bias ([heads * key_dim]), norm ([value_dim])."""
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} q/k heads")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.key_dim, self.value_dim, self.taps = int(key_dim), int(value_dim), int(taps)
        self.decay_rank, self.gate_rank = int(decay_rank), int(gate_rank)
        self.norm_eps = float(norm_eps)
        self.names = dict(names)
        qk, v = num_kv_heads * key_dim, num_heads * value_dim
        self.channels = 2 * qk + v
        # one product for everything that reads h: q | k | v | a1 | g1 | b
        self.inp = Linear(hidden_size, [names[x] for x in ("q", "k", "v", "a1", "g1", "b")],
                          [qk, qk, v, self.decay_rank, self.gate_rank, num_heads])
        self.col_a1 = self.channels
        self.col_g1 = self.col_a1 + self.decay_rank
        self.col_b = self.col_g1 + self.gate_rank
        # the second halves of the two low-rank projections as one product: the weight is [a2 0; 0 g2], its input
        # the neighbouring columns a1 | g1 of the stacked product (zeros add nothing to a 32-bit sum)
        self.low = Linear(self.decay_rank + self.gate_rank, [f"{names['a2']}+{names['g2']}"], [num_heads * key_dim + v])
        self.out = Linear(v, [names["o"]], [hidden_size])
        self.conv_w = self.a_log = self.dt_bias = self.norm_w = None

    def tensor_specs(self) -> list[TensorSpec]:
        n, qk, v = self.names, self.num_kv_heads * self.key_dim, self.num_heads * self.value_dim
        return (self.inp.tensor_specs() + self.out.tensor_specs() + [
            TensorSpec(n["a2"], (self.num_heads * self.key_dim, self.decay_rank), MATRIX),
            TensorSpec(n["g2"], (v, self.gate_rank), MATRIX),
            TensorSpec(n["q_conv"], (qk, self.taps), CONV),
            TensorSpec(n["k_conv"], (qk, self.taps), CONV),
            TensorSpec(n["v_conv"], (v, self.taps), CONV),
            TensorSpec(n["A_log"], (self.num_heads,), VECTOR),
            TensorSpec(n["dt_bias"], (self.num_heads * self.key_dim,), VECTOR),
            TensorSpec(n["norm"], (self.value_dim,), NORM_WEIGHT),
        ])

    def state_need(self) -> StateNeed:
        return StateNeed((ops.delta_state_size(self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim, self.taps),),
                         torch.float32)

    def load(self, tensors: dict[str, torch.Tensor], placer: Placer) -> None:
        for lin in (self.inp, self.out):
            lin.load(tensors, placer)
        n = self.names

        def block_diagonal() -> torch.Tensor:
            a2, g2 = tensors[n["a2"]], tensors[n["g2"]]
            w = torch.zeros((a2.shape[0] + g2.shape[0], a2.shape[1] + g2.shape[1]), dtype=placer.dtype)
            w[: a2.shape[0], : a2.shape[1]] = a2.to(placer.dtype)
            w[a2.shape[0] :, a2.shape[1] :] = g2.to(placer.dtype)
            return w.contiguous().to(placer.device)

        self.low.weight = placer.place(("block_diagonal", n["a2"], n["g2"]), block_diagonal)

        def f32(key: tuple, make) -> torch.Tensor:
            return placer.place(key, lambda: make().to(torch.float32).contiguous().to(placer.device))

        self.conv_w = f32(("conv_f32", n["q_conv"], n["k_conv"], n["v_conv"]),
                          lambda: torch.cat([tensors[n["q_conv"]], tensors[n["k_conv"]], tensors[n["v_conv"]]], dim=0))
        self.a_log = f32(("vector_f32", n["A_log"]), lambda: tensors[n["A_log"]])
        self.dt_bias = f32(("vector_f32", n["dt_bias"]), lambda: tensors[n["dt_bias"]])
        self.norm_w = f32(("vector_f32", n["norm"]), lambda: tensors[n["norm"]])

    @staticmethod
    def _columns(x: torch.Tensor, first: int, count: int) -> torch.Tensor:
        """Columns of the stacked product as an operand of the next: a view when its rows start
        at multiples of 16 bytes, else a copy."""
        part = x[:, first : first + count]
        if x.dtype == torch.float32 or (first % 8 == 0 and count % 8 == 0 and x.stride(0) % 8 == 0):
            return part
        # (a new buffer: a one-row view counts as contiguous whatever its stride says)
        return torch.empty((x.shape[0], count), dtype=x.dtype, device=x.device).copy_(part)

    def _run(self, h: torch.Tensor, ctx: StepContext, state: torch.Tensor, rows: torch.Tensor | None) -> torch.Tensor:
        assert state is not None, "the delta rule keeps its state in the request's slot"
        H, G, dk, dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        proj = self.inp(h)
        low = self.low(self._columns(proj, self.col_a1, self.decay_rank + self.gate_rank), out_f32=True)
        a_pre, gate = low[:, : H * dk], low[:, H * dk :]  # 32-bit, rows a stride apart
        rec = ops.delta_prepare(proj, self.col_b, a_pre, self.conv_w, self.a_log, self.dt_bias, state,
                                ctx.q_start, ctx.token_req, ctx.slots, H, G, dk, dv)
        o = ops.delta_rule(rec, state, ctx.q_start, ctx.slots, H, G, dk, dv)
        y = ops.gated_head_norm(o, gate, self.norm_w, self.norm_eps, H, dv, h.dtype)
        return y if rows is None else ops.gather_rows(y, rows)

    def mix(self, h, ctx, cache, state, rows, out_f32: bool = False):
        return self.out(self._run(h, ctx, state, rows), out_f32=out_f32)

    def forward(self, h, residual, ctx, cache, state, rows):
        return self.out(self._run(h, ctx, state, rows), residual=residual)
