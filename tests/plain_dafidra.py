"""A plain, slow implementation of the Dafidra forward pass: whole sequences, no cache, no
batching, one function per mechanism, explicit loops over positions and heads on the CPU in
float64.  It shares no code with ``photon_infer_amd`` and reads a model folder by itself.

Notation: T tokens at positions 0 .. T-1, h [T, D] a sublayer's input, rows of weight matrices
are outputs (y = W h).  ``act_round`` (optional) rounds activations where a bfloat16 engine
rounds them (a sublayer's input, the attention's queries / keys / values, weights and output, the
memory's output before its projection, the gated product), which gives tests a yardstick for
the bfloat16 path; None rounds nothing.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional

import torch

from plain_llama import bf16_round, read_model_folder  # noqa: F401  (file reading and rounding only)

F = torch.float64
Round = Optional[Callable[[torch.Tensor], torch.Tensor]]


def _r(t: torch.Tensor, act_round: Round) -> torch.Tensor:
    return act_round(t.to(torch.float32)).to(F) if act_round is not None else t


def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float, offset: float = 0.0) -> torch.Tensor:
    """Row by row: x / sqrt(mean(x^2) + eps) * (offset + w); w None: no weight."""
    out = torch.empty_like(x)
    for t in range(x.shape[0]):
        out[t] = x[t] / math.sqrt(float((x[t] * x[t]).sum()) / x.shape[1] + eps)
        if w is not None:
            out[t] = out[t] * (offset + w)
    return out


def query_temperature(p: int, coef: float, every: int) -> float:
    return 1.0 + coef * math.log((p + 1) // every + 1)


def distance_slope(head: int, heads: int) -> float:
    return 2.0 ** (-8.0 * (head + 1) / heads)


def sink_softmax(scores: List[float], sink: Optional[float]) -> List[float]:
    """exp(s_j) / (sum_j exp(s_j) + exp(sink)); sink None: the usual softmax."""
    top = max(scores + ([sink] if sink is not None else []))
    e = [math.exp(s - top) for s in scores]
    den = sum(e) + (math.exp(sink - top) if sink is not None else 0.0)
    return [v / den for v in e]


def sink_window_attention(h: torch.Tensor, W: Dict[str, torch.Tensor], c: dict, eps: float, act_round: Round = None) -> torch.Tensor:
    """The left mixer; ``W`` holds its tensors by their names after the mixer's prefix."""
    T = h.shape[0]
    H, G, d, dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    window = c["mask"]["size"] if c.get("mask") else None
    temp = c.get("q_temp")
    q = rms_norm(h @ W["q"].T, W["q.norm"], eps)       # over the whole projection, all heads at once
    k = rms_norm(h @ W["k"].T, W["k.norm"], eps)
    v = h @ W["v"].T
    gate = torch.sigmoid(h @ W["g"].T)
    if temp:
        for p in range(T):
            q[p] = q[p] * query_temperature(p, temp["coef"], temp["every"])
    q, k, v = _r(q, act_round), _r(k, act_round), _r(v, act_round)
    out = torch.zeros(T, H * dv, dtype=F)
    for n in range(H):
        g = n // (H // G)
        for i in range(T):
            lo = 0 if window is None else max(0, i - window + 1)
            scores = [float(q[i, n * d:(n + 1) * d] @ k[j, g * d:(g + 1) * d]) * c["scale"] - distance_slope(n, H) * (i - j)
                      for j in range(lo, i + 1)]
            probs = sink_softmax(scores, float(W["sink"][n]))
            if act_round is not None:      # a bfloat16 engine may round the weights for their product with the values
                probs = _r(torch.tensor(probs, dtype=F), act_round).tolist()
            acc = torch.zeros(dv, dtype=F)
            for j, p in zip(range(lo, i + 1), probs):
                acc += p * v[j, g * dv:(g + 1) * dv]
            out[i, n * dv:(n + 1) * dv] = acc * gate[i, n]
    return _r(out, act_round) @ W["o"].T


def log_sigmoid(x: float) -> float:
    return min(x, 0.0) - math.log1p(math.exp(-abs(x)))


def matrix_memory(h: torch.Tensor, W: Dict[str, torch.Tensor], c: dict, eps: float, act_round: Round = None) -> torch.Tensor:
    """The right mixer: the recurrence token by token from a zero state."""
    T = h.shape[0]
    H, d, dv, cap = c["heads"], c["dim"], c["vdim"], c["gate_cap"]
    q = (h @ W["q"].T) * d ** -0.5
    k, v = h @ W["k"].T, h @ W["v"].T
    zi, zf = h @ W["i"].T + W["i.b"], h @ W["f"].T + W["f.b"]
    cell = torch.zeros(T, H * dv, dtype=F)
    for n in range(H):
        S, nv, m = torch.zeros(d, dv, dtype=F), torch.zeros(d, dtype=F), 0.0
        for t in range(T):
            i_t = cap * math.tanh(float(zi[t, n]) / cap)
            f_t = log_sigmoid(cap * math.tanh(float(zf[t, n]) / cap))
            m_new = max(f_t + m, i_t)
            a, b = math.exp(f_t + m - m_new), math.exp(i_t - m_new)
            kt, vt, qt = k[t, n * d:(n + 1) * d], v[t, n * dv:(n + 1) * dv], q[t, n * d:(n + 1) * d]
            S = a * S + b * torch.outer(kt, vt)
            nv = a * nv + b * kt
            m = m_new
            o = (S.T @ qt) / (max(abs(float(nv @ qt)), math.exp(-m)) + 1e-6)
            cell[t, n * dv:(n + 1) * dv] = o / math.sqrt(float((o * o).sum()) / dv + eps)
    y = cell * W["norm"] * torch.sigmoid(h @ W["g"].T)
    return _r(y, act_round) @ W["o"].T


def gated_ffn(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, act_round: Round = None) -> torch.Tensor:
    g, u = _r(h @ gate.T, act_round), _r(h @ up.T, act_round)       # a bfloat16 engine may store the two products before it gates
    return _r(g * torch.sigmoid(g) * u, act_round) @ down.T


def route(z: torch.Tensor, top: int, groups: int, keep: int):
    """One token's router logits -> [(expert, weight)]: softmax over all experts; only experts of
    the ``keep`` groups with the largest best score may be chosen; the weights are the scores."""
    s = torch.softmax(z, dim=-1).tolist()
    E = len(s)
    per = E // groups
    order = sorted(range(groups), key=lambda g: (-max(s[g * per:(g + 1) * per]), g))[:keep]
    allowed = [e for e in range(E) if e // per in order]
    chosen = sorted(allowed, key=lambda e: (-s[e], e))[:top]
    return [(e, s[e]) for e in chosen]


def route_margin(z: torch.Tensor, top: int, groups: int, keep: int) -> float:
    """How far (in logits) the token is from another choice: the smaller of the gap between the last
    expert chosen and the best allowed one left out, and the gap between the last group kept and the
    best group dropped.  Tests use it to stay away from close calls, which rounding may decide either way."""
    zs = z.tolist()
    E = len(zs)
    per = E // groups
    best = sorted(((max(zs[g * per:(g + 1) * per]), g) for g in range(groups)), reverse=True)
    margin = best[keep - 1][0] - best[keep][0] if keep < groups else float("inf")
    kept = {g for _, g in best[:keep]}
    allowed = sorted((zs[e] for e in range(E) if e // per in kept), reverse=True)
    if top < len(allowed):
        margin = min(margin, allowed[top - 1] - allowed[top])
    return margin


def routed_experts(h: torch.Tensor, W: Dict[str, torch.Tensor], c: dict, act_round: Round = None, margins: Optional[list] = None,
                   forced=None, chosen: Optional[list] = None) -> torch.Tensor:
    """``forced`` ([T, top] expert ids): use these experts instead of the router's own choice, each with its own
    score (for comparisons with an engine whose rounding decided a close call the other way); ``chosen`` receives
    the router's own choice per token."""
    r = c["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    out = torch.zeros_like(h)
    z = h @ W["router"].T
    for t in range(h.shape[0]):
        if margins is not None:
            margins.append(route_margin(z[t], r["top"], g["count"], g["keep"]))
        own = route(z[t], r["top"], g["count"], g["keep"])
        if chosen is not None:
            chosen.append([e for e, _ in own])
        if forced is not None:
            s = torch.softmax(z[t], dim=-1)
            own = [(int(e), float(s[int(e)])) for e in forced[t]]
        for e, w in own:
            out[t] += w * gated_ffn(h[t:t + 1], W[f"e{e}.gate"], W[f"e{e}.up"], W[f"e{e}.down"], act_round)[0]
    return out


def _sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {n[len(prefix):]: t.to(F) for n, t in tensors.items() if n.startswith(prefix)}


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], act_round: Round = None, streams: Optional[list] = None,
            margins: Optional[list] = None, forced: Optional[dict] = None, chosen: Optional[dict] = None):
    """float64 logits [T, vocab] of a whole sequence; ``streams`` (a list) receives the residual stream after every layer,
    ``margins`` (a list) every routing decision's margin (``route_margin``); ``forced`` / ``chosen``: per routed layer
    (by layer index) the experts to use / the router's own choices, see ``routed_experts``."""
    eps, m = config["norm"]["eps"], config["residual_mult"]
    x = torch.stack([tensors["embed"][int(t)].to(F) for t in tokens])
    for i, layer in enumerate(config["layers"]):
        assert layer["type"] == "parallel"
        p = f"l{i}."
        h = _r(x, act_round)
        a = sink_window_attention(h, _sub(tensors, p + "mix.left."), layer["mixer"]["left"], eps, act_round)
        b = matrix_memory(h, _sub(tensors, p + "mix.right."), layer["mixer"]["right"], eps, act_round)
        mix = 0.5 * (rms_norm(a, tensors[p + "mix.left.out"].to(F), eps) + rms_norm(b, tensors[p + "mix.right.out"].to(F), eps))
        x = x + m * rms_norm(mix, tensors[p + "norm1"].to(F), eps, 1.0)
        if layer["mlp"] is not None:
            h = _r(x, act_round)
            W = _sub(tensors, p + "mlp.")
            f = gated_ffn(h, W["gate"], W["up"], W["down"], act_round) if layer["mlp"]["kind"] == "dense" else routed_experts(
                h, W, layer["mlp"], act_round, margins if margins is None else margins.setdefault(i, []) if isinstance(margins, dict) else margins,
                forced.get(i) if forced else None, chosen.setdefault(i, []) if chosen is not None else None)
            x = x + m * rms_norm(f, tensors[p + "norm2"].to(F), eps, 1.0)
        if streams is not None:
            streams.append(x.clone())
    return _r(rms_norm(x, tensors["final.norm"].to(F), eps, 1.0), act_round) @ tensors["head"].to(F).T


def greedy_generate(config: dict, tensors, prompt: List[int], n_new: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(torch.argmax(forward(config, tensors, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out
