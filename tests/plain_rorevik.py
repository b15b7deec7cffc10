"""Plain implementation of the Rorevik design: whole sequences, no cache, float64, loops over
positions and heads, one function per mechanism.  It shares nothing with the engine: it takes
the raw config.json mapping and a dict of tensors by their names in a model folder.

    x_0 = norm(embed[token] * scale + pos[p]; embed.norm)
    per layer run:  x <- x + mixer(norm(x; norm1));  x <- x + ff(norm(x; norm2))   (layers with a feed-forward)
    logits = head . norm(x; final.norm)

The layers ``loop.start .. loop.stop - 1`` run ``loop.times`` times in a row (same weights, a
state or cache per pass), then the rest follow.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) [* w] over the last axis."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def causal_conv(u: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u [T, C]; w [C, taps], the last column weighs the current token; zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    out = torch.zeros((T, C), dtype=F64)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] += w[:, j] * u[src]
        if b is not None:
            out[t] += b
    return out


def rotate_interleaved(x: torch.Tensor, pos: int, dims: int, base: float) -> torch.Tensor:
    """x [heads, dim]: pairs (2i, 2i+1), i < dims / 2, turned by pos * base^(-2i / dims); the rest unchanged."""
    y = x.clone()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, v = x[:, 2 * i].clone(), x[:, 2 * i + 1].clone()
        y[:, 2 * i] = u * c - v * s
        y[:, 2 * i + 1] = v * c + u * s
    return y


def softcap_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], m: dict) -> torch.Tensor:
    """Causal grouped-query attention with partly rotated heads and capped scores.  h [T, D] -> [T, D]."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W["q"].T).view(T, H, d)
    k = (h @ W["k"].T).view(T, G, d)
    v = (h @ W["v"].T).view(T, G, dv)
    rot = m.get("rot")
    if rot is not None:
        q = torch.stack([rotate_interleaved(q[t], t, rot["dims"], rot["base"]) for t in range(T)])
        k = torch.stack([rotate_interleaved(k[t], t, rot["dims"], rot["base"]) for t in range(T)])
    cap = m.get("softcap")
    out = torch.zeros((T, H, dv), dtype=F64)
    for i in range(T):
        for n in range(H):
            g = n // (H // G)
            s = (k[: i + 1, g] @ q[i, n]) * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            p = torch.softmax(s, dim=0)
            out[i, n] = p @ v[: i + 1, g]
    return out.reshape(T, H * dv) @ W["o"].T


def state_space(h: torch.Tensor, W: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """The state-space mixer (Mamba-2 form).  h [T, D] -> [T, D]."""
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ W["in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner: 2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W["conv"], W["conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner: inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + W["dt_bias"])
    y = torch.zeros((T, H, P), dtype=F64)
    for n in range(H):
        g = n // (H // G)
        S = torch.zeros((N, P), dtype=F64)
        for t in range(T):
            S = torch.exp(-torch.exp(W["A_log"][n]) * dt[t, n]) * S + dt[t, n] * torch.outer(B[t, g], x[t, n])
            y[t, n] = S.T @ C[t, g] + W["D"][n] * x[t, n]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms_norm(y.view(T, parts, inner // parts), None, eps).reshape(T, inner) * W["norm"]
    return y @ W["o"].T


def channel_delta(h: torch.Tensor, W: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """The gated delta rule with one decay per head and key channel.  h [T, D] -> [T, D]."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ W["q"].T, W["q.conv"])).view(T, G, d)
    k = silu(causal_conv(h @ W["k"].T, W["k.conv"])).view(T, G, d)
    v = silu(causal_conv(h @ W["v"].T, W["v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W["b"].T)                                           # [T, H]
    a = (h @ W["a1"].T) @ W["a2"].T + W["dt_bias"]
    decay = torch.exp(-torch.exp(W["A_log"]).view(1, H, 1) * softplus(a).view(T, H, d))
    gate = torch.sigmoid((h @ W["g1"].T) @ W["g2"].T).view(T, H, dv)
    o = torch.zeros((T, H, dv), dtype=F64)
    for n in range(H):
        g = n // (H // G)
        S = torch.zeros((d, dv), dtype=F64)
        for t in range(T):
            S = decay[t, n].view(d, 1) * S
            u = beta[t, n] * (v[t, n] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, n] = S.T @ q[t, g]
    o = rms_norm(o, W["norm"], eps) * gate
    return o.reshape(T, H * dv) @ W["o"].T


def clamped_glu(h: torch.Tensor, W: Dict[str, torch.Tensor], limit: float) -> torch.Tensor:
    g = torch.clamp(h @ W["gate"].T + W["gate.b"], max=limit)
    u = torch.clamp(h @ W["up"].T + W["up.b"], min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W["down"].T + W["down.b"]


def sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {n[len(prefix):]: t.to(F64) for n, t in tensors.items() if n.startswith(prefix)}


def run_order(config: dict) -> List[int]:
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def mixer(h: torch.Tensor, tensors, layer: dict, prefix: str, eps: float) -> torch.Tensor:
    m = layer["mixer"]
    if layer["type"] == "parallel":
        left = softcap_attention(h, sub(tensors, prefix + "mix.left."), m["left"])
        right = state_space(h, sub(tensors, prefix + "mix.right."), m["right"], eps)
        return m["left_scale"] * left + m["right_scale"] * right
    if layer["type"] == "channel_delta":
        return channel_delta(h, sub(tensors, prefix + "mix."), m, eps)
    raise ValueError(layer["type"])


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens, streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] (float64) of one whole sequence; ``streams`` collects the stream after every layer run."""
    eps = config["norm"]["eps"]
    T = len(tokens)
    f = lambda n: tensors[n].to(F64)
    x = f("embed")[torch.as_tensor(list(tokens))] * config["embedding"]["scale"] + f("pos")[:T]
    x = rms_norm(x, f("embed.norm"), eps)
    for i in run_order(config):
        layer, prefix = config["layers"][i], f"l{i}."
        x = x + mixer(rms_norm(x, f(prefix + "norm1"), eps), tensors, layer, prefix, eps)
        if layer.get("mlp") is not None:
            x = x + clamped_glu(rms_norm(x, f(prefix + "norm2"), eps), sub(tensors, prefix + "mlp."), layer["mlp"]["limit"])
        if streams is not None:
            streams.append(x.clone())
    return rms_norm(x, f("final.norm"), eps) @ f("head").T


def greedy(config: dict, tensors, prompt, new_tokens: int) -> List[int]:
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(torch.argmax(forward(config, tensors, tokens)[-1])))
    return tokens[len(prompt):]
