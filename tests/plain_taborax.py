"""A plain, slow Taborax on whole sequences, one function per mechanism, written from the
equations alone.  It shares no code with the engine: tensors by their checkpoint names, the
configuration as the dict that config.json holds, everything in the dtype of the weights it is
given (float64 for an oracle).

Notation: T tokens, W the width, H query heads, G key heads, d the query/key size of a head,
dv its value size, r the size of the key/value latent, E routed experts, I identity experts.
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def squared_relu(z):
    return torch.relu(z) ** 2


# --------------------------------------------------------------------------- mixers


def causal_scores(q: torch.Tensor, k: torch.Tensor, scale: float) -> torch.Tensor:
    """q [T, H, d], k [T, H, d] -> scores [H, T, T] with -inf above the diagonal."""
    s = torch.einsum("ihd,jhd->hij", q, k) * scale
    T = q.shape[0]
    hidden = torch.ones(T, T, dtype=torch.bool).triu(1)
    return s.masked_fill(hidden, -math.inf)


def softmax_with_unit_sink(s: torch.Tensor) -> torch.Tensor:
    """p_j = exp(s_j) / (1 + sum_j exp(s_j)): one more score of 0 that carries no value."""
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, rot: dict | None) -> torch.Tensor:
    """x [T, heads, d]: of the leading ``dims`` elements of a head, element i and element
    i + dims/2 are a pair turned by the angle position * base^(-2i/dims); the rest passes."""
    if not rot:
        return x
    dims = int(rot["dims"])
    half = dims // 2
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    a = positions.to(torch.float64)[:, None] * f[None, :]
    c, s = torch.cos(a).to(x.dtype)[:, None, :], torch.sin(a).to(x.dtype)[:, None, :]
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def shared_kv_attention(h, w, p, mixer, positions):
    """Grouped-query attention whose values are its keys as projected (unrotated), rotary
    positions on queries and keys, and a unit sink in the softmax."""
    H, G, d = mixer["heads"], mixer["kv_heads"], mixer["dim"]
    T = h.shape[0]
    q = (h @ w[f"{p}.q"].T).view(T, H, d)
    k = (h @ w[f"{p}.k"].T).view(T, G, d)
    v = k
    q = rotate_halves(q, positions, mixer.get("rot"))
    k = rotate_halves(k, positions, mixer.get("rot"))
    each = H // G
    k_of_head = k.repeat_interleave(each, dim=1)
    v_of_head = v.repeat_interleave(each, dim=1)
    pr = softmax_with_unit_sink(causal_scores(q, k_of_head, float(mixer["scale"])))
    o = torch.einsum("hij,jhd->ihd", pr, v_of_head).reshape(T, H * mixer["vdim"])
    return o @ w[f"{p}.o"].T


def latent_attention(h, w, p, mixer, eps):
    """Queries through a normed latent; keys and values expanded per head from one normed
    latent a token; no positions; ordinary softmax."""
    H, d, dv = mixer["heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    cq = norm(h @ w[f"{p}.dq"].T, w[f"{p}.dq.norm"], eps)
    q = (cq @ w[f"{p}.uq"].T).view(T, H, d)
    c = norm(h @ w[f"{p}.dkv"].T, w[f"{p}.dkv.norm"], eps)
    k = (c @ w[f"{p}.uk"].T).view(T, H, d)
    v = (c @ w[f"{p}.uv"].T).view(T, H, dv)
    pr = torch.softmax(causal_scores(q, k, float(mixer["scale"])), dim=-1)
    o = torch.einsum("hij,jhd->ihd", pr, v).reshape(T, H * dv)
    return o @ w[f"{p}.o"].T


# --------------------------------------------------------------------------- feed-forwards


def dense_ff(h, w, p):
    return squared_relu(h @ w[f"{p}.up"].T) @ w[f"{p}.down"].T


def gated_expert(h, w, p):
    return (silu(h @ w[f"{p}.gate"].T) * (h @ w[f"{p}.up"].T)) @ w[f"{p}.down"].T


def route(h, w, p, router):
    """For every token the chosen experts and their weights.  Softmax over routed and identity
    experts together; the choice is by score + correction, only inside the best groups of
    neighbours (a group's mark is its best choice score); the weight is the score itself."""
    E, I, top = int(router["experts"]), int(router.get("identity") or 0), int(router["top"])
    groups = router.get("groups") or {"count": 1, "keep": 1}
    s = torch.softmax(h @ w[f"{p}.router"].T, dim=-1)  # [T, E + I]
    choice = s + w[f"{p}.correction"]
    n = E + I
    per = n // int(groups["count"])
    marks = choice.view(-1, int(groups["count"]), per).max(-1).values
    kept = marks.topk(int(groups["keep"]), dim=-1).indices
    open_ = torch.zeros_like(marks, dtype=torch.bool).scatter_(1, kept, True).repeat_interleave(per, dim=1)
    chosen = choice.masked_fill(~open_, -math.inf).topk(top, dim=-1).indices
    return chosen, s.gather(1, chosen)


def mixture_ff(h, w, p, mlp):
    router = mlp["router"]
    E = int(router["experts"])
    chosen, weight = route(h, w, p, router)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weight[t]):
            y = gated_expert(h[t : t + 1], w, f"{p}.e{e}")[0] if e < E else h[t]
            out[t] += g * y
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ w[f"{p}.shared.sg"].T) * gated_expert(h, w, f"{p}.shared")
    return out


# --------------------------------------------------------------------------- the model


def run_order(cfg: dict) -> list[int]:
    """Layer indices in the order they run: layers start .. stop-1 ``times`` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def layer(x, w, cfg, i, positions):
    spec, eps, p = cfg["layers"][i], float(cfg["norm"]["eps"]), f"l{i}"
    h = norm(x, w[f"{p}.norm1"], eps)
    if spec["type"] == "latent_attention":
        y = latent_attention(h, w, f"{p}.mix", spec["mixer"], eps)
    elif spec["type"] == "attention":
        y = shared_kv_attention(h, w, f"{p}.mix", spec["mixer"], positions)
    else:
        raise ValueError(spec["type"])
    x = x + norm(y, w[f"{p}.norm1b"], eps)
    mlp = spec.get("mlp")
    if mlp is None:
        return x
    h = norm(x, w[f"{p}.norm2"], eps)
    y = dense_ff(h, w, f"{p}.mlp") if mlp["kind"] == "dense" else mixture_ff(h, w, f"{p}.mlp", mlp)
    return x + norm(y, w[f"{p}.norm2b"], eps)


def forward(tokens: list[int], w: dict, cfg: dict, streams: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence; ``streams`` collects the stream after every layer run."""
    positions = torch.arange(len(tokens))
    x0 = w["embed"][torch.tensor(tokens)]
    x = x0
    loop = cfg.get("loop")
    first_of_pass = int(loop["start"]) if loop else None
    for i in run_order(cfg):
        if loop and i == first_of_pass:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T
        x = layer(x, w, cfg, i, positions)
        if streams is not None:
            streams.append(x.clone())
    return norm(x, w["final.norm"], float(cfg["norm"]["eps"])) @ w["head"].T
