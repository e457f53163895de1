"""A layer whose sub-layers stand between two norms, around a residual stream kept in 32-bit:

    x <- x + norm_b(mixer(norm_a(x)));   x <- x + norm_d(ffn(norm_c(x)))          (a layer may lack the feed-forward)

The stream that this arrangement hands from block to block is the 32-bit array [tokens, width].  One kernel does what
stands between two sub-layers (`ops.sandwich_step`): it norms the output of the one that has run, adds it, and forms the
normed input of the next; a block therefore leaves its last output un-added (`PostNormed`) for the first kernel of the
block behind it, or for the model's end.  What a looped range of layers lets into the stream before a pass
(`ctx.pass_input`: rows and a vector) enters through the same kernel, behind the sum and before the norm.
`enter` makes the stream from the embedding's rows and `leave` turns the wanted rows into the final norm's output, so
the model's own two ends stay as they are.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from .. import ops
from ..config.spec import LayerSpec, SpecError
from ..weights.loader import TensorSpec
from .base import BlockBase, part_class, register_block
from .block import sub_tensors


@dataclass
class PostNormed:
    """A sub-layer's output that is not in the stream yet: y (or `y_scale` y + `y2_scale` y2) goes through `norm` first."""
    y: torch.Tensor
    norm: object
    y_scale: float = 1.0
    y2: Optional[torch.Tensor] = None
    y2_scale: float = 1.0

    def args(self) -> dict:
        return dict(y=self.y, y_scale=self.y_scale, y2=self.y2, y2_scale=self.y2_scale, post_weight=self.norm.weight,
                    post_eps=self.norm.eps)


def _post(out, norm) -> PostNormed:
    if isinstance(out, ops.state.WeightedPair):
        return PostNormed(out.left, norm, out.left_scale, out.right, out.right_scale)
    if hasattr(out, "materialize"):
        out = out.materialize()
    return PostNormed(out, norm)


@register_block("sandwich_norm")
class SandwichBlock(BlockBase):

    @classmethod
    def tensors(cls, spec: LayerSpec) -> Dict[str, TensorSpec]:
        n_norms = 2 if spec.ffn is None else 4
        if len(spec.norms) != n_norms or len(spec.norm_names) != n_norms:
            raise SpecError(f"the arrangement 'sandwich_norm' has {n_norms} norms here, the layer names {len(spec.norms)}")
        out: Dict[str, TensorSpec] = {}
        for local, ts in part_class("mixer", spec.mixer).tensors(spec.mixer).items():
            out[spec.mixer_prefix + local] = ts
        if spec.ffn is not None:
            for local, ts in part_class("ffn", spec.ffn).tensors(spec.ffn).items():
                out[spec.ffn_prefix + local] = ts
        for name, nspec in zip(spec.norm_names, spec.norms):
            (ts,) = part_class("norm", nspec).tensors(nspec).values()
            out[name] = ts
        return out

    def __init__(self, spec: LayerSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec, self.dtype = spec, dtype
        self.mixer = part_class("mixer", spec.mixer)(spec.mixer, sub_tensors(tensors, spec.mixer_prefix), dtype, device)
        self.ffn = None
        if spec.ffn is not None:
            self.ffn = part_class("ffn", spec.ffn)(spec.ffn, sub_tensors(tensors, spec.ffn_prefix), dtype, device)
        self.norms = [part_class("norm", nspec)(nspec, {"weight": tensors[name]}, dtype, device)
                      for name, nspec in zip(spec.norm_names, spec.norms)]
        if len(self.norms) != (2 if self.ffn is None else 4):
            raise SpecError("sandwich_norm: a norm before and a norm behind every sub-layer")
        for n in self.norms:
            if getattr(n, "add_one", False) or not hasattr(n, "weight") or not hasattr(n, "eps"):
                raise SpecError("sandwich_norm: the norms must be plain RMS norms")
        self.first_norm = self.norms[0]

    def parts(self):
        return [self.mixer, self.ffn, *self.norms, getattr(self.mixer, "position", None),
                *getattr(self.mixer, "parts", lambda: [])()]

    # ---- the model's two ends ---------------------------------------------------------------------
    def enter(self, ctx, rows: torch.Tensor) -> torch.Tensor:
        """The embedding's rows -> the 32-bit stream (a copy: the rows themselves may enter again later)."""
        return ops.widen(rows) if rows.dtype == torch.bfloat16 else rows.clone()

    def leave(self, ctx, x: torch.Tensor, pending, rows: torch.Tensor, norm) -> torch.Tensor:
        """The final norm of the wanted rows, with what the last block left to be added."""
        if norm is None or getattr(norm, "add_one", False):
            raise SpecError("sandwich_norm: the model ends with a plain RMS norm")
        return ops.sandwich_step(x, rows=rows, pre_weight=norm.weight, eps=norm.eps, h_dtype=self.dtype,
                                 **self._pending(pending))

    @staticmethod
    def _pending(pending) -> dict:
        if pending is None:
            return {}
        if not isinstance(pending, PostNormed):
            raise SpecError("sandwich_norm: the block before leaves something that this arrangement does not take")
        return pending.args()

    # ---- a layer ------------------------------------------------------------------------------------
    def forward(self, ctx, x: torch.Tensor, pending, cache, next_norm=None) -> Tuple[torch.Tensor, object]:
        if x.dim() != 2 or x.dtype != torch.float32:
            raise SpecError(f"sandwich_norm: the block takes a 32-bit stream [tokens, width], got {tuple(x.shape)} {x.dtype}")
        ctx.stream = ctx.stream_norm = None
        ctx.partial_sums = False
        enter = {}
        if getattr(ctx, "pass_input", None) is not None:
            enter = dict(enter_rows=ctx.pass_input[0], enter_vector=ctx.pass_input[1])
            ctx.pass_input = None
        h = ops.sandwich_step(x, pre_weight=self.norms[0].weight, eps=self.norms[0].eps, h_dtype=self.dtype,
                              **self._pending(pending), **enter)
        a = _post(self.mixer.forward(ctx, h, cache), self.norms[1])
        if self.ffn is None:
            return x, a
        h2 = ops.sandwich_step(x, pre_weight=self.norms[2].weight, eps=self.norms[2].eps, h_dtype=self.dtype, **a.args())
        return x, _post(self.ffn.forward(ctx, h2), self.norms[3])
