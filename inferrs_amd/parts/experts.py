"""Routed experts: a router scores every expert for a token, the `top` best run, and their outputs are added up
with score * scale as weights.  An expert: g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit),
W_down (g * sigmoid(alpha g) * (u + 1)).  The router's logits are 32-bit.

`forward` returns `RoutedRows`: one 32-bit output row a (token, chosen expert) and the weights; whoever adds the
feed-forward's output to the stream adds them up, a token's rows in the order of its choice, so a token's sum does
not depend on the other tokens of the step (`.materialize()` gives the plain sum for a block that knows nothing of
this)."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import RoutedExpertsSpec, SpecError
from ..weights.loader import TensorSpec
from .base import FeedForward, register_ffn
from .linear import to_compute


class RoutedRows:
    """rows [n, top, width] (32-bit) and weights [n, top] (32-bit): the output is sum_k weights[:, k] * rows[:, k]."""
    __slots__ = ("rows", "weights")

    def __init__(self, rows: torch.Tensor, weights: torch.Tensor):
        self.rows, self.weights = rows, weights

    def materialize(self) -> torch.Tensor:
        n, top, width = self.rows.shape
        streams = torch.zeros((n, 1, width), dtype=torch.float32, device=self.rows.device)
        one = torch.ones((1,), dtype=torch.float32, device=self.rows.device)
        ops.streams_step(streams, y=self.rows, y_weights=self.weights, mix=one, out=one)
        return streams.view(n, width)


@register_ffn("routed_experts")
class RoutedExperts(FeedForward):
    graph_safe = True

    @classmethod
    def tensors(cls, spec: RoutedExpertsSpec) -> Dict[str, TensorSpec]:
        t = {"router": TensorSpec((spec.experts, spec.hidden))}
        for e in range(spec.experts):
            t[f"e{e}.gate"] = TensorSpec((spec.intermediate, spec.hidden))
            t[f"e{e}.up"] = TensorSpec((spec.intermediate, spec.hidden))
            t[f"e{e}.down"] = TensorSpec((spec.hidden, spec.intermediate))
        return t

    def __init__(self, spec: RoutedExpertsSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        if not (1 <= spec.top <= spec.experts <= ops.mix.MAX_EXPERTS) or spec.top > ops.mix.MAX_TOP:
            raise SpecError(f"routed_experts: top {spec.top} of {spec.experts} experts (up to {ops.mix.MAX_TOP} of {ops.mix.MAX_EXPERTS})")
        if spec.score not in ops.mix.SCORE_FUNCTIONS:
            raise SpecError(f"routed_experts: score {spec.score!r} has no kernel (known: {sorted(ops.mix.SCORE_FUNCTIONS)})")
        self.spec = spec
        # the router's logits are 32-bit sums whatever its matrix is stored in (`ops.route`)
        self.router = to_compute(tensors["router"], dtype, device)
        E = spec.experts
        gate_up = torch.stack([torch.cat([to_compute(tensors[f"e{e}.gate"], dtype, device),
                                          to_compute(tensors[f"e{e}.up"], dtype, device)], dim=0) for e in range(E)])
        down = torch.stack([to_compute(tensors[f"e{e}.down"], dtype, device) for e in range(E)])
        # bfloat16 experts whose sizes the matrix cores take keep their weights as tiles of 64 features x 64 inputs
        self.tiled = ops.mix.experts_tiled_fits(dtype, spec.hidden, spec.intermediate)
        if self.tiled:
            gate_up = ops.mix.tile_weights(gate_up.view(E, 2, spec.intermediate, spec.hidden))
            down = ops.mix.tile_weights(down)
        self.gate_up, self.down = gate_up.contiguous(), down.contiguous()

    def forward(self, ctx, h):
        s = self.spec
        sel, weights = ops.route(h, self.router, s.top, s.scale, s.score, s.renormalize)
        return RoutedRows(ops.experts_forward(h, sel, self.gate_up, self.down, s.limit, s.alpha,
                                              ff=s.intermediate if self.tiled else None), weights)
