"""Rorevik: a pre-norm decoder whose layers hold either two mixers side by side - attention with
partly rotated heads and capped scores, and a state-space mixer - or a delta-rule memory with a
decay per key channel; a span of layers may run several times in a row.

    x = norm(embed[token] * scale + pos[p]; embed.norm)
    per layer run:  x <- x + mixer(norm(x; norm1));  x <- x + ffn(norm(x; norm2))     (layers with a feed-forward)
    logits = head . norm(x; final.norm)

    mixer of a "parallel" layer:       left_scale * attention(h) + right_scale * state_space(h)
    mixer of a "channel_delta" layer:  the delta rule with channel-wise decay

The layers ``loop.start .. loop.stop - 1`` run ``loop.times`` times in a row with the same weights,
every pass with a cache or state of its own (the run order names a layer once per pass).  Layer i's
tensors start with ``l<i>.``; the mixers' with ``mix.`` (``mix.left.`` / ``mix.right.``), the
feed-forward's with ``mlp.``; norms are named by themselves (``l<i>.norm1``, ``final.norm``).
"""
from __future__ import annotations

from ..config.rorevik import ChannelDeltaConfig, ParallelMixerConfig, RorevikConfig
from ..errors import UnsupportedModelError
from ..parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS
from ..parts.embedding import LMHead, PositionedEmbedding
from ..parts.model import ModelSpec, RunEntry
from ..registry import register_architecture


def _mixer(cfg: RorevikConfig, m, ropes: dict):
    D, eps = cfg.width, cfg.norm_eps
    if isinstance(m, ParallelMixerConfig):
        a, r = m.left, m.right
        rope = None
        if a.rot_dims:
            # layers that rotate alike share the part, and with it a step's table of cosines and sines
            key = (a.dim, a.rot_dims, a.rot_base)
            if key not in ropes:
                ropes[key] = POSITION_ENCODINGS.make("rope", head_dim=a.dim, theta=a.rot_base, interleaved=True, rotary_dim=a.rot_dims)
            rope = ropes[key]
        left = MIXERS.make("attention", hidden_size=D, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim, position=rope,
                           scale=a.scale, value_dim=a.vdim, softcap=a.softcap, out_scale=m.left_scale, names=("q", "k", "v", "o"), any_head_size=True)
        right = MIXERS.make("state_space", hidden_size=D, num_heads=r.heads, value_dim=r.vdim, state_dim=r.state, groups=r.groups,
                            norm_groups=r.norm_groups, conv_taps=r.conv, eps=eps, out_scale=m.right_scale)
        return MIXERS.make("side_by_side", branches=[("left.", left), ("right.", right)])
    if isinstance(m, ChannelDeltaConfig):
        if m.decay_rank is None or m.gate_rank is None:
            raise UnsupportedModelError("the delta rule's low-rank sizes are open: a model folder gives them by its tensors "
                                        "(registry.load_config), a bare configuration names 'decay_rank' and 'gate_rank'")
        return MIXERS.make("channel_delta_rule", hidden_size=D, num_heads=m.heads, num_kv_heads=m.kv_heads, key_dim=m.dim,
                           value_dim=m.vdim, conv_taps=m.conv, decay_rank=m.decay_rank, gate_rank=m.gate_rank, eps=eps)
    raise UnsupportedModelError(f"no mixer for {type(m).__name__}")


def build_rorevik(cfg: RorevikConfig) -> ModelSpec:
    D, eps = cfg.width, cfg.norm_eps
    norm = lambda: NORMS.make("rmsnorm", dim=D, eps=eps, tensor_name="")
    layers, ignorable, ropes = [], [], {}
    for i, layer in enumerate(cfg.layers):
        norm2 = ffn = None
        if layer.mlp is not None:
            norm2 = ("norm2", norm())
            ffn = ("mlp.", FEED_FORWARDS.make("clamped_glu", hidden_size=D, intermediate_size=layer.mlp.ff, limit=layer.mlp.limit))
        else:
            ignorable.append(f"l{i}.norm2")      # a layer without a feed-forward has no use for its norm
        block = BLOCKS.make("prenorm", norm1=("norm1", norm()), mixer=("mix.", _mixer(cfg, layer.mixer, ropes)), norm2=norm2, ffn=ffn)
        layers.append((f"l{i}.", block))
    embedding = PositionedEmbedding(cfg.vocab, D, cfg.max_positions, scale=cfg.embedding_scale, norm=("embed.norm", norm()),
                                    tensor_name="embed", position_name="pos")
    return ModelSpec(
        hidden_size=D, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=("", embedding), layers=layers, run_order=[RunEntry(i) for i in cfg.run_order()],
        final_norm=("final.norm", norm()), head=("head", LMHead(cfg.vocab, D, tied=False, tensor_name="")),
        ignorable=tuple(ignorable),
    )


register_architecture("Rorevik", RorevikConfig, build_rorevik)
