"""A recurrent mixer with a matrix memory per head: the mLSTM cell of xLSTM (Beck et al.,
"xLSTM: Extended Long Short-Term Memory").

Per head, with input h: ``q = Wq h * d^(-1/2)``, ``k = Wk h`` (size d), ``v = Wv h`` (size dv),
log gates ``i = cap * tanh((Wi h + bi) / cap)`` and ``f = logsigmoid(cap * tanh((Wf h + bf) / cap))``.
State S [d, dv], n [d] and a running maximum m, all zero at the start of a sequence:

    m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' likewise with k alone;
    o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)

Each head's o is divided by its root mean square, the heads are concatenated and multiplied by
a weight ``norm`` and by ``sigmoid(Wg h)``, then projected by ``Wo``.  Gates, state and the cell
are float32 in both compute modes; the state lives in the request's slot and is carried from
step to step, so a prompt may be cut anywhere.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import MIXERS, LayerCache, Mixer, StateSpec, StepContext


class MatrixMemory(Mixer):
    graph_safe = True        # slots and request boundaries are read on the device

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, gate_cap: float, eps: float,
                 accumulate: bool = True):
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.gate_cap, self.eps = float(gate_cap), float(eps)
        self.accumulate = bool(accumulate)     # False: forward writes its result instead of adding it
        self.qk_size, self.v_size = self.num_heads * self.key_dim, self.num_heads * self.value_dim

    def tensor_specs(self) -> List[TensorSpec]:
        D, H = self.hidden_size, self.num_heads
        return [TensorSpec("q", (self.qk_size, D)), TensorSpec("k", (self.qk_size, D)), TensorSpec("v", (self.v_size, D)),
                TensorSpec("g", (self.v_size, D)), TensorSpec("o", (D, self.v_size)), TensorSpec("norm", (self.v_size,), "norm"),
                TensorSpec("i", (H, D)), TensorSpec("i.b", (H,), "bias"), TensorSpec("f", (H, D)), TensorSpec("f.b", (H,), "bias")]

    def cache_spec(self):
        return StateSpec((ops.matrix_memory_state_floats(self.num_heads, self.key_dim, self.value_dim),), torch.float32)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        # one projection, rows [q | k | v | g | i | f]
        self.w_in = torch.cat([tensors[n] for n in ("q", "k", "v", "g", "i", "f")], dim=0).contiguous()
        QK, V, H = self.qk_size, self.v_size, self.num_heads
        self.offsets = (0, QK, 2 * QK, 2 * QK + 2 * V, 2 * QK + 2 * V + H)     # q, k, v, i, f
        self.g_offset = 2 * QK + V
        self.w_o = tensors["o"]
        f32 = lambda t: t.to(torch.float32).contiguous()
        self.w_norm, self.i_bias, self.f_bias = f32(tensors["norm"]), f32(tensors["i.b"]), f32(tensors["f.b"])

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T, ws = h.shape[0], ctx.workspace
        proj = torch.empty((T, self.w_in.shape[0]), dtype=torch.float32, device=h.device)
        ops.gemm(proj, h, self.w_in, ws=ws)
        cell = torch.empty((T, self.v_size), dtype=torch.float32, device=h.device)
        ops.matrix_memory_scan(cell, proj, self.offsets, self.i_bias, self.f_bias, self.gate_cap, self.key_dim ** -0.5, ctx,
                               cache.state, self.num_heads, self.key_dim, self.value_dim)
        y = torch.empty((T, self.v_size), dtype=self.dtype, device=h.device)
        ops.head_norm_gate(y, cell, proj[:, self.g_offset:self.g_offset + self.v_size], self.w_norm, self.eps,
                           self.num_heads, self.value_dim)
        ops.gemm(x, y, self.w_o, accumulate=self.accumulate,
                 may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


MIXERS.register("matrix_memory", MatrixMemory)
