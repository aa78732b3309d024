"""A plain, slow Kupuzen on whole sequences, one function per mechanism, written from the
equations alone.  It shares no code with the engine: tensors by their checkpoint names, the
configuration as the dict that config.json holds, everything in the dtype of the weights it is
given (float64 for an oracle).

Notation: T tokens, W the width, H query (or value) heads, G key heads, dk / dv the key and
value sizes of a head.
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return rms(x, eps) * (1.0 + w)


def silu(z):
    return z * torch.sigmoid(z)


def rotary_frequencies(rot: dict | None, dtype=torch.float64) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims/2, with the three bands of wavelength scaling (none for no rotation)."""
    if not rot:
        return torch.zeros(0, dtype=dtype)
    dims = int(rot["dims"])
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for fi in f.tolist():
            wavelength = 2.0 * math.pi / fi
            if wavelength < orig / high:
                out.append(fi)
            elif wavelength > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wavelength - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = torch.tensor(out, dtype=torch.float64)
    return f.to(dtype)


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """x [T, heads, d]: elements 2i and 2i+1 of the leading 2 * len(freqs) are a pair turned by
    the angle position * f_i; the rest passes."""
    n = freqs.numel()
    a = positions.to(freqs.dtype)[:, None] * freqs[None, :]  # [T, n]
    c, s = torch.cos(a).to(x.dtype)[:, None, :], torch.sin(a).to(x.dtype)[:, None, :]
    out = x.clone()
    u, v = x[..., 0 : 2 * n : 2], x[..., 1 : 2 * n : 2]
    out[..., 0 : 2 * n : 2] = u * c - v * s
    out[..., 1 : 2 * n : 2] = v * c + u * s
    return out


def attention_keys_values(h, w, p, mixer, eps, positions):
    """Keys (normed over the whole projection, rotated) [T, G, dk] and values [T, G, dv]."""
    G, dk, dv = mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    k = h @ w[f"{p}.k"].T
    k = rms(k, eps) * w[f"{p}.k.norm"]
    k = rotate_interleaved(k.view(-1, G, dk), positions, rotary_frequencies(mixer.get("rot"), h.dtype))
    v = (h @ w[f"{p}.v"].T).view(-1, G, dv)
    return k, v


def attention(h, w, p, mixer, eps, positions, kv=None):
    """Sliding-window attention with a sink in the softmax's denominator.  ``kv``: keys and
    values of another layer to use in place of this layer's own."""
    H, G, dk, dv = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    q = h @ w[f"{p}.q"].T
    q = rms(q, eps) * w[f"{p}.q.norm"]
    q = rotate_interleaved(q.view(T, H, dk), positions, rotary_frequencies(mixer.get("rot"), h.dtype))
    k, v = kv if kv is not None else attention_keys_values(h, w, p, mixer, eps, positions)
    window = mixer.get("mask", {}).get("size") if mixer.get("mask") else None
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(mixer["scale"])  # [T, T]
        i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
        seen = (j <= i) if window is None else ((i - j >= 0) & (i - j < window))
        s = s.masked_fill(~seen, float("-inf"))
        sink = w[f"{p}.sink"][hd]
        m = torch.maximum(s.max(-1).values, sink)
        e = torch.exp(s - m[:, None])
        out[:, hd] = (e / (e.sum(-1) + torch.exp(sink - m))[:, None]) @ v[:, g]
    return out.reshape(T, H * dv) @ w[f"{p}.o"].T, (k, v)


def short_conv(x, taps_w):
    """x [T, C], taps_w [C, taps]: y_t = sum_j taps_w[:, j] * x_{t - (taps - 1) + j}, zeros before 0."""
    T, C = x.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x])
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + padded[j : j + T] * taps_w[:, j][None, :]
    return y


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def channel_delta(h, w, p, mixer, eps):
    """Gated delta rule with one decay per head and key channel."""
    H, G, dk, dv = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    q = silu(short_conv(h @ w[f"{p}.q"].T, w[f"{p}.q.conv"])).view(T, G, dk)
    k = silu(short_conv(h @ w[f"{p}.k"].T, w[f"{p}.k.conv"])).view(T, G, dk)
    v = silu(short_conv(h @ w[f"{p}.v"].T, w[f"{p}.v.conv"])).view(T, H, dv)
    q, k = unit(q) * dk**-0.5, unit(k)
    beta = torch.sigmoid(h @ w[f"{p}.b"].T)  # [T, H]
    pre = (h @ w[f"{p}.a1"].T) @ w[f"{p}.a2"].T + w[f"{p}.dt_bias"]
    decay = torch.exp(-torch.exp(w[f"{p}.A_log"])[None, :, None] * torch.nn.functional.softplus(pre).view(T, H, dk))
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(dk, dv, dtype=h.dtype)
        for t in range(T):
            S = decay[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hd] = S.T @ q[t, g]
    gate = torch.sigmoid((h @ w[f"{p}.g1"].T) @ w[f"{p}.g2"].T).view(T, H, dv)
    o = rms(o, eps) * w[f"{p}.norm"] * gate
    return o.reshape(T, H * dv) @ w[f"{p}.o"].T


def dense_ff(h, w, p):
    return (silu(h @ w[f"{p}.gate"].T) * (h @ w[f"{p}.up"].T)) @ w[f"{p}.down"].T


def forward(config: dict, w: dict, tokens: list[int], return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the stream after every layer)."""
    eps = float(config["norm"]["eps"])
    m = float(config["residual_mult"])
    x = w["embed"][torch.tensor(tokens)] * float(config["embedding"]["scale"])
    positions = torch.arange(len(tokens))
    kept: dict[int, tuple] = {}
    streams = []
    for i, layer in enumerate(config["layers"]):
        p, mixer = f"l{i}.mix", layer["mixer"]
        h1 = offset_norm(x, w[f"l{i}.norm1"], eps)
        if layer["type"] == "attention":
            src = mixer.get("kv_from")
            y, kept[i] = attention(h1, w, p, mixer, eps, positions, kv=None if src is None else kept[src])
        elif layer["type"] == "channel_delta":
            y = channel_delta(h1, w, p, mixer, eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp"):
            y = y + dense_ff(offset_norm(x, w[f"l{i}.norm2"], eps), w, f"l{i}.mlp")
        x = x + m * y
        streams.append(x)
    logits = offset_norm(x, w["final.norm"], eps) @ w["head"].T
    cap = config.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return (logits, torch.stack(streams)) if return_layers else logits
