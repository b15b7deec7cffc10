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

import json
import math
import os
from typing import Callable, Dict, List, Optional

import torch

F64 = torch.float64
Round = Optional[Callable[[torch.Tensor], torch.Tensor]]


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype)


def _r(t: torch.Tensor, act_round: Round) -> torch.Tensor:
    """Activations rounded where an engine that computes in a 16-bit type rounds them (None: not at all)."""
    return act_round(t.to(torch.float32)).to(F64) if act_round is not None else t


def read_model_folder(model_dir: str):
    """(raw config.json, tensors by name) of a model folder written with safetensors."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json"), encoding="utf-8") as f:
        config = json.load(f)
    return config, load_file(os.path.join(model_dir, "model.safetensors"))


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


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, cap: Optional[float]) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence -> [T, H, dv]: position i sees every j <= i;
    the scaled score s becomes cap * tanh(s / cap); ordinary softmax."""
    T, H, G = q.shape[0], q.shape[1], k.shape[1]
    out = torch.zeros((T, H, v.shape[2]), dtype=F64)
    for i in range(T):
        for n in range(H):
            g = n // (H // G)
            s = (k[: i + 1, g] @ q[i, n]) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            out[i, n] = torch.softmax(s, dim=0) @ v[: i + 1, g]
    return out


def softcap_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], m: dict, act_round: Round = None) -> torch.Tensor:
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
    q, k, v = _r(q, act_round), _r(k, act_round), _r(v, act_round)
    out = attend(q, k, v, m["scale"], m.get("softcap"))
    return _r(out.reshape(T, H * dv) * m.get("out_scale", 1.0), act_round) @ W["o"].T


def state_space_recurrence(x, B, C, dt, A_log, D, S0=None):
    """x [T, H, P], B and C [T, G, N], dt [T, H] (after softplus): S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x.
    Returns (y [T, H, P], the states after the last token [H, N, P])."""
    T, H, P = x.shape
    G, N = B.shape[1], B.shape[2]
    y, last = torch.zeros((T, H, P), dtype=F64), []
    for n in range(H):
        g = n // (H // G)
        S = torch.zeros((N, P), dtype=F64) if S0 is None else S0[n].clone()
        for t in range(T):
            S = torch.exp(-torch.exp(A_log[n]) * dt[t, n]) * S + dt[t, n] * torch.outer(B[t, g], x[t, n])
            y[t, n] = S.T @ C[t, g] + D[n] * x[t, n]
        last.append(S)
    return y, torch.stack(last)


def delta_recurrence(q, k, v, beta, decay, S0=None):
    """q and k [T, G, d] (unit vectors; q scaled), v [T, H, dv], beta [T, H], decay [T, H, d]:
    S <- diag(decay) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  Returns (o [T, H, dv], states [H, d, dv])."""
    T, H, dv = v.shape
    G, d = k.shape[1], k.shape[2]
    o, last = torch.zeros((T, H, dv), dtype=F64), []
    for n in range(H):
        g = n // (H // G)
        S = torch.zeros((d, dv), dtype=F64) if S0 is None else S0[n].clone()
        for t in range(T):
            S = decay[t, n].view(d, 1) * S
            u = beta[t, n] * (v[t, n] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, n] = S.T @ q[t, g]
        last.append(S)
    return o, torch.stack(last)


def unit(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def state_space(h: torch.Tensor, W: Dict[str, torch.Tensor], m: dict, eps: float, act_round: Round = None) -> torch.Tensor:
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
    y, _ = state_space_recurrence(x, B, C, softplus(dt + W["dt_bias"]), W["A_log"], W["D"])
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms_norm(y.view(T, parts, inner // parts), None, eps).reshape(T, inner) * W["norm"]
    return _r(y * m.get("out_scale", 1.0), act_round) @ W["o"].T


def channel_delta(h: torch.Tensor, W: Dict[str, torch.Tensor], m: dict, eps: float, act_round: Round = None) -> torch.Tensor:
    """The gated delta rule with one decay per head and key channel.  h [T, D] -> [T, D]."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ W["q"].T, W["q.conv"])).view(T, G, d)
    k = silu(causal_conv(h @ W["k"].T, W["k.conv"])).view(T, G, d)
    v = silu(causal_conv(h @ W["v"].T, W["v.conv"])).view(T, H, dv)
    q, k = unit(q) * d ** -0.5, unit(k)
    beta = torch.sigmoid(h @ W["b"].T)                                           # [T, H]
    a = _r(h @ W["a1"].T, act_round) @ W["a2"].T + W["dt_bias"]
    decay = torch.exp(-torch.exp(W["A_log"]).view(1, H, 1) * softplus(a).view(T, H, d))
    gate = torch.sigmoid(_r(h @ W["g1"].T, act_round) @ W["g2"].T).view(T, H, dv)
    o, _ = delta_recurrence(q, k, v, beta, decay)
    o = rms_norm(o, W["norm"], eps) * gate
    return _r(o.reshape(T, H * dv), act_round) @ W["o"].T


def clamped_glu(h: torch.Tensor, W: Dict[str, torch.Tensor], limit: float, act_round: Round = None, alpha: float = 1.702) -> torch.Tensor:
    g = torch.clamp(h @ W["gate"].T + W["gate.b"], max=limit)
    u = torch.clamp(h @ W["up"].T + W["up.b"], min=-limit, max=limit)
    return _r(g * torch.sigmoid(alpha * g) * (u + 1.0), act_round) @ W["down"].T + W["down.b"]


def sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {n[len(prefix):]: t.to(F64) for n, t in tensors.items() if n.startswith(prefix)}


def run_order(config: dict) -> List[int]:
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def mixer(h: torch.Tensor, tensors, layer: dict, prefix: str, eps: float, act_round: Round = None) -> torch.Tensor:
    m = layer["mixer"]
    if layer["type"] == "parallel":
        # an engine that rounds activations applies a branch's factor before the rounding in front of its output projection
        if act_round is not None:
            left = softcap_attention(h, sub(tensors, prefix + "mix.left."), dict(m["left"], out_scale=m["left_scale"]), act_round)
            right = state_space(h, sub(tensors, prefix + "mix.right."), dict(m["right"], out_scale=m["right_scale"]), eps, act_round)
            return left + right
        left = softcap_attention(h, sub(tensors, prefix + "mix.left."), m["left"])
        right = state_space(h, sub(tensors, prefix + "mix.right."), m["right"], eps)
        return m["left_scale"] * left + m["right_scale"] * right
    if layer["type"] == "channel_delta":
        return channel_delta(h, sub(tensors, prefix + "mix."), m, eps, act_round)
    raise ValueError(layer["type"])


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens, streams: Optional[list] = None,
            act_round: Round = None) -> torch.Tensor:
    """Logits [T, vocab] (float64) of one whole sequence; ``streams`` collects the stream after every layer run;
    ``act_round`` rounds activations where a 16-bit engine does (the stream itself never)."""
    eps = config["norm"]["eps"]
    T = len(tokens)
    f = lambda n: tensors[n].to(F64)
    x = f("embed")[torch.as_tensor(list(tokens))] * config["embedding"]["scale"] + f("pos")[:T]
    x = rms_norm(x, f("embed.norm"), eps)
    for i in run_order(config):
        layer, prefix = config["layers"][i], f"l{i}."
        x = x + mixer(_r(rms_norm(x, f(prefix + "norm1"), eps), act_round), tensors, layer, prefix, eps, act_round)
        if layer.get("mlp") is not None:
            x = x + clamped_glu(_r(rms_norm(x, f(prefix + "norm2"), eps), act_round), sub(tensors, prefix + "mlp."),
                                layer["mlp"]["limit"], act_round)
        if streams is not None:
            streams.append(x.clone())
    return _r(rms_norm(x, f("final.norm"), eps), act_round) @ f("head").T


def greedy(config: dict, tensors, prompt, new_tokens: int) -> List[int]:
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(torch.argmax(forward(config, tensors, tokens)[-1])))
    return tokens[len(prompt):]
