"""Routed experts (mixture of experts) feed-forward.

Router logits ``z = Wr h`` in float32; scores ``s = softmax(z)`` over all experts.  Experts form
``groups`` equal groups of neighbours; a group's score is its largest expert score and only
experts of the ``keep`` best groups can be chosen.  Each token uses the ``top`` allowed experts
with the largest scores, weighted by those scores as they are (``renormalize``: divided by
their sum).  An expert is a gated feed-forward ``Wdown (silu(Wgate h) * (Wup h))`` without
biases; the result is the weighted sum of the chosen experts' outputs (float32).

The step's (token, choice) entries are sorted by expert on the device and each expert's rows go
through grouped products; nothing is counted on the host.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import FEED_FORWARDS, FeedForward, StepContext
from .mlp import INTERLEAVE


class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, groups: int = 1, keep: int = 1,
                 renormalize: bool = False, activation: str = "silu", accumulate: bool = True,
                 expert_prefix: str = "e", names=("gate", "up", "down"), router_name: str = "router"):
        if activation != "silu":
            raise UnsupportedModelError(f"expert activation '{activation}' is not supported")
        self.hidden_size, self.expert_size = int(hidden_size), int(expert_size)
        self.num_experts, self.top, self.groups, self.keep = int(num_experts), int(top), int(groups), int(keep)
        if not 0 < self.top <= self.num_experts:
            raise UnsupportedModelError(f"routed experts: {self.top} choices among {self.num_experts} experts")
        if self.groups > 1 and (self.num_experts % self.groups or not 0 < self.keep <= self.groups
                                or self.keep * (self.num_experts // self.groups) < self.top):
            raise UnsupportedModelError(f"routed experts: {self.num_experts} experts in {self.groups} groups of which {self.keep} "
                                        f"are kept cannot give {self.top} choices")
        self.renormalize, self.accumulate = bool(renormalize), bool(accumulate)
        self.expert_prefix, self.names, self.router_name = expert_prefix, tuple(names), router_name

    def tensor_specs(self) -> List[TensorSpec]:
        F, D = self.expert_size, self.hidden_size
        specs = []
        for e in range(self.num_experts):
            p = f"{self.expert_prefix}{e}."
            specs += [TensorSpec(p + self.names[0], (F, D)), TensorSpec(p + self.names[1], (F, D)), TensorSpec(p + self.names[2], (D, F))]
        specs.append(TensorSpec(self.router_name, (self.num_experts, D)))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        E, p = self.num_experts, self.expert_prefix
        F, b = self.expert_size, INTERLEAVE
        mats = []
        for e in range(E):
            g, u = tensors[f"{p}{e}.{self.names[0]}"], tensors[f"{p}{e}.{self.names[1]}"]
            if g.dtype == torch.bfloat16 and u.dtype == torch.bfloat16 and F % b == 0:
                # gate and up rows interleaved in blocks of 16, as the dense gated feed-forward keeps them: the
                # matrix-core product then applies the activation before anything is stored
                mats.append(torch.stack([g.view(F // b, b, -1), u.view(F // b, b, -1)], dim=1).reshape(2 * F, -1))
            else:
                mats.append(torch.cat([g, u], dim=0))
        self.interleave = b if all(t.dtype == torch.bfloat16 for t in mats) and F % b == 0 else 0
        self.w_gate_up = torch.stack(mats).contiguous()                   # [E, 2F, D]
        self.w_down = torch.stack([tensors[f"{p}{e}.{self.names[2]}"] for e in range(E)]).contiguous()   # [E, D, F]
        self.tile = ops.grouped_tile_rows(self.w_gate_up.dtype if self.w_down.dtype == self.w_gate_up.dtype else torch.float32)
        self.w_router = tensors[self.router_name]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        T, ws = h.shape[0], ctx.workspace if ctx is not None else None
        logits = torch.empty((T, self.num_experts), dtype=torch.float32, device=h.device)
        ops.gemm(logits, h, self.w_router, ws=ws)
        ids, weights = ops.route(logits, self.top, self.groups, self.keep, self.renormalize)
        rows = ops.group_entries(ids, self.num_experts, self.tile)
        a = ops.gather_rows(h, rows)
        act = torch.empty((rows.rows, self.expert_size), dtype=self.dtype, device=h.device)
        ops.grouped_gemm_swiglu(act, a, self.w_gate_up, rows, self.interleave)
        y = torch.empty((rows.rows, self.hidden_size), dtype=torch.float32, device=h.device)
        ops.grouped_gemm(y, act, self.w_down, rows)
        if self.accumulate:
            ops.materialize(x, ws)
        ops.combine_choices(x, y, weights, rows, accumulate=self.accumulate)


FEED_FORWARDS.register("routed_experts", RoutedExperts)
