"""A state-space mixer in the Mamba-2 form (Dao and Gu, "Transformers are SSMs: Generalized
Models and Efficient Algorithms Through Structured State Space Duality").

With input h, ``inner = heads * value_dim``, N = ``state_dim``, G = ``groups``:

* one projection ``W_in h`` laid out ``[z: inner | x: inner | B: G N | C: G N | dt: heads]``;
* x, B and C together pass a causal convolution per channel (``conv`` [channels, taps], the last
  column on the current token, bias ``conv.b``, zeros before the start of a sequence) and silu;
* ``dt <- softplus(dt + dt_bias)``; per head n with group ``n // (heads / G)`` and state S [N, value_dim]:
  ``S <- exp(-exp(A_log_n) dt) S + dt B x^T``, ``y = S^T C + D_n x``;
* ``y * silu(z)``, RMS-normalised in ``norm_groups`` equal parts with the weight ``norm`` (the gate
  comes before the norm), times ``out_scale``, then ``W_o``.

Steps, decays, the state and the norm are float32 in both compute modes.  A request's state row
holds the convolution's last taps - 1 inputs and S, is cleared when the request is admitted and
carried from step to step, so a prompt may be cut anywhere.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import MIXERS, LayerCache, Mixer, StateSpec, StepContext


class StateSpaceMixer(Mixer):
    graph_safe = True        # slots and request boundaries are read on the device

    def __init__(self, hidden_size: int, num_heads: int, value_dim: int, state_dim: int, groups: int, norm_groups: int,
                 conv_taps: int, eps: float, out_scale: float = 1.0, accumulate: bool = True):
        self.hidden_size, self.num_heads, self.value_dim = int(hidden_size), int(num_heads), int(value_dim)
        self.state_dim, self.groups, self.norm_groups, self.conv_taps = int(state_dim), int(groups), int(norm_groups), int(conv_taps)
        self.eps, self.out_scale, self.accumulate = float(eps), float(out_scale), bool(accumulate)
        self.inner = self.num_heads * self.value_dim
        self.channels = self.inner + 2 * self.groups * self.state_dim          # what the convolution sees: x | B | C
        self.proj_size = 2 * self.inner + 2 * self.groups * self.state_dim + self.num_heads
        if self.num_heads % self.groups or self.inner % self.norm_groups:
            raise UnsupportedModelError(f"state space: {self.num_heads} heads in {self.groups} groups, {self.inner} columns in "
                                        f"{self.norm_groups} norm parts")
        if not 1 <= self.conv_taps <= ops.CONV_MAX_TAPS or self.state_dim > 256:
            raise UnsupportedModelError(f"state space: {self.conv_taps} taps (at most {ops.CONV_MAX_TAPS}), state of {self.state_dim} (at most 256)")
        self.conv_floats = (self.conv_taps - 1) * self.channels

    def tensor_specs(self) -> List[TensorSpec]:
        D, H = self.hidden_size, self.num_heads
        return [TensorSpec("in", (self.proj_size, D)), TensorSpec("conv", (self.channels, self.conv_taps), "taps"),
                TensorSpec("conv.b", (self.channels,), "small_bias"), TensorSpec("dt_bias", (H,), "bias"), TensorSpec("A_log", (H,), "bias"),
                TensorSpec("D", (H,), "bias"), TensorSpec("norm", (self.inner,), "norm"), TensorSpec("o", (D, self.inner))]

    def cache_spec(self):
        return StateSpec((self.conv_floats + ops.scan_state_floats(self.num_heads, self.state_dim, self.value_dim),), torch.float32)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        self.w_in, self.w_o = tensors["in"], tensors["o"]
        self.w_conv, self.b_conv = tensors["conv"].contiguous(), tensors["conv.b"].to(tensors["conv"].dtype).contiguous()
        f32 = lambda t: t.to(torch.float32).contiguous()
        self.dt_bias, self.a_log, self.skip, self.w_norm = f32(tensors["dt_bias"]), f32(tensors["A_log"]), f32(tensors["D"]), f32(tensors["norm"])

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T, ws, inner = h.shape[0], ctx.workspace, self.inner
        proj = torch.empty((T, self.proj_size), dtype=torch.float32, device=h.device)
        ops.gemm(proj, h, self.w_in, ws=ws)
        xbc = torch.empty((T, self.channels), dtype=torch.float32, device=h.device)
        ops.causal_conv_silu(xbc, proj[:, inner:inner + self.channels], self.w_conv, self.b_conv, ctx, cache.state[:, :self.conv_floats])
        y = torch.empty((T, inner), dtype=torch.float32, device=h.device)
        ops.state_space_scan(y, xbc, proj[:, inner + self.channels:], self.dt_bias, self.a_log, self.skip, ctx,
                             cache.state[:, self.conv_floats:], self.num_heads, self.value_dim, self.state_dim, self.groups)
        act = torch.empty((T, inner), dtype=self.dtype, device=h.device)
        ops.gated_group_norm(act, y, proj[:, :inner], self.w_norm, self.eps, self.norm_groups, self.out_scale)
        ops.gemm(x, act, self.w_o, accumulate=self.accumulate,
                 may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


MIXERS.register("state_space", StateSpaceMixer)
