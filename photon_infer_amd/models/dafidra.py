"""Dafidra: a decoder whose layers hold two mixers side by side - windowed attention with a sink
and a distance bias, and a matrix memory - normalised on the way out, and a dense or routed
feed-forward.

    x = embed[token]
    per layer:  x <- x + m * norm1((norm(left(x); left.out) + norm(right(x); right.out)) / 2)
                x <- x + m * norm2(ffn(x))                      (layers with a feed-forward)
    logits = head . norm(x; final.norm)

``norm1``, ``norm2`` and ``final.norm`` store their weights around zero (used as 1 + w); the two
branch norms have plain weights.  Layer i's tensors start with ``l<i>.``; the mixers' with
``mix.left.`` / ``mix.right.``, the feed-forward's with ``mlp.``.
"""
from __future__ import annotations

from ..config.dafidra import DafidraConfig
from ..parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS
from ..parts.embedding import LMHead, TokenEmbedding
from ..parts.model import ModelSpec
from ..registry import register_architecture


def build_dafidra(cfg: DafidraConfig) -> ModelSpec:
    D, eps = cfg.width, cfg.norm_eps
    plain = lambda: NORMS.make("rmsnorm", dim=D, eps=eps, tensor_name="")
    one_plus = lambda: NORMS.make("rmsnorm", dim=D, eps=eps, offset=1.0, tensor_name="")
    layers, ignorable = [], []
    for i, layer in enumerate(cfg.layers):
        a, r = layer.left, layer.right
        left = MIXERS.make("sink_window_attention", hidden_size=D, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim,
                           value_dim=a.vdim, scale=a.scale, window=a.window, eps=eps, temp_coef=a.temp_coef,
                           temp_every=a.temp_every, accumulate=False)
        right = MIXERS.make("matrix_memory", hidden_size=D, num_heads=r.heads, key_dim=r.dim, value_dim=r.vdim,
                            gate_cap=r.gate_cap, eps=eps, accumulate=False)
        ffn = norm2 = None
        if layer.mlp is not None:
            norm2 = ("norm2", one_plus())
            if layer.mlp.kind == "dense":
                ffn = FEED_FORWARDS.make("swiglu", hidden_size=D, intermediate_size=layer.mlp.ff, names=("gate", "up", "down"),
                                         accumulate=False)
            else:
                ffn = FEED_FORWARDS.make("routed_experts", hidden_size=D, expert_size=layer.mlp.ff, num_experts=layer.mlp.experts,
                                         top=layer.mlp.top, groups=layer.mlp.groups, keep=layer.mlp.keep, accumulate=False)
            ffn = ("mlp.", ffn)
        else:
            ignorable.append(f"l{i}.norm2")      # a layer without a feed-forward has no use for its norm
        block = BLOCKS.make("output_norm",
                            branches=[("mix.left.", left, ("mix.left.out", plain())), ("mix.right.", right, ("mix.right.out", plain()))],
                            norm1=("norm1", one_plus()), mult=cfg.residual_mult, norm2=norm2, ffn=ffn)
        layers.append((f"l{i}.", block))
    return ModelSpec(
        hidden_size=D, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=("embed", TokenEmbedding(cfg.vocab, D, tensor_name="")), layers=layers,
        final_norm=("final.norm", one_plus()), head=("head", LMHead(cfg.vocab, D, tied=False, tensor_name="")),
        ignorable=tuple(ignorable),
    )


register_architecture("Dafidra", DafidraConfig, build_dafidra)
