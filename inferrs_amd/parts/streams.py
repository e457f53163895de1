"""A pre-norm layer around several residual streams (hyper-connections), kept in 32-bit.

Every token has S streams x_1..x_S, all equal to the embedding's row at the start.  Sub-layer q of a layer (1: the
mixer, 2: the feed-forward, which a layer may lack) reads u = sum_s in_q[s] x_s through its RMS norm; its output y is
scaled feature by feature (`ls<q>`), and the streams become, all at once from the old ones,

    x_t <- sum_s mix_q[s, t] x_s + out_q[t] * y.

At the model's end the streams are added up.  One kernel does what stands between two sub-layers: it adds the
output of the one that has run and forms the normed input of the next (`ops.streams_step`).  Without learned
connections (`StreamsSpec.connections` False) every coefficient is 1: with one stream that is the ordinary residual
sum, in 32-bit, with a layer scale.

The stream that this arrangement hands from block to block is the 32-bit array [tokens, S, width]; `enter` makes
it from the embedding's rows and `leave` turns the wanted rows into the final norm's output, so the model's own two
ends stay as they are.
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from .. import ops
from ..config.spec import LayerSpec, SpecError, StreamsSpec
from ..weights.loader import TensorSpec
from .base import BlockBase, part_class, register_block
from .block import sub_tensors


def _names(res: StreamsSpec, q: int):
    p = res.prefix
    return f"{p}hc{q}.in", f"{p}hc{q}.out", f"{p}hc{q}.mix", f"{p}ls{q}"


@register_block("streams")
class StreamsBlock(BlockBase):

    @classmethod
    def tensors(cls, spec: LayerSpec) -> Dict[str, TensorSpec]:
        res: StreamsSpec = spec.residual
        n_sub = 1 if spec.ffn is None else 2
        if res is None or len(spec.norms) != n_sub or len(spec.norm_names) != n_sub:
            raise SpecError("the arrangement 'streams' needs a StreamsSpec and one norm for every sub-layer")
        out: Dict[str, TensorSpec] = {}
        for local, ts in part_class("mixer", spec.mixer).tensors(spec.mixer).items():
            out[spec.mixer_prefix + local] = ts
        if spec.ffn is not None:
            for local, ts in part_class("ffn", spec.ffn).tensors(spec.ffn).items():
                out[spec.ffn_prefix + local] = ts
        for name, nspec in zip(spec.norm_names, spec.norms):
            (ts,) = part_class("norm", nspec).tensors(nspec).values()
            out[name] = ts
        for q in range(1, n_sub + 1):
            n_in, n_out, n_mix, n_ls = _names(res, q)
            if res.connections:
                out[n_in] = TensorSpec((res.streams,), "norm")
                out[n_out] = TensorSpec((res.streams,), "norm")
                out[n_mix] = TensorSpec((res.streams, res.streams), "eye")
            if res.layer_scale:
                out[n_ls] = TensorSpec((res.hidden,), "norm")
        return out

    def __init__(self, spec: LayerSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        res: StreamsSpec = spec.residual
        if not (1 <= res.streams <= ops.mix.MAX_STREAMS):
            raise SpecError(f"streams: {res.streams} residual streams (1..{ops.mix.MAX_STREAMS})")
        if not res.connections and res.streams != 1:
            raise SpecError("streams: several streams need their connections")
        self.spec, self.res, self.dtype = spec, res, dtype
        self.mixer = part_class("mixer", spec.mixer)(spec.mixer, sub_tensors(tensors, spec.mixer_prefix), dtype, device)
        self.ffn = None
        if spec.ffn is not None:
            self.ffn = part_class("ffn", spec.ffn)(spec.ffn, sub_tensors(tensors, spec.ffn_prefix), dtype, device)
        self.norms = [part_class("norm", nspec)(nspec, {"weight": tensors[name]}, dtype, device)
                      for name, nspec in zip(spec.norm_names, spec.norms)]
        for n in self.norms:
            if getattr(n, "add_one", False) or not hasattr(n, "weight") or not hasattr(n, "eps"):
                raise SpecError("streams: the sub-layers' norms must be plain RMS norms")
        self.first_norm = self.norms[0]

        def f32(name, shape):
            return tensors[name].to(device=device, dtype=torch.float32).reshape(shape).contiguous()

        S = res.streams
        self.coef = []                          # for every sub-layer: (in, out, mix, layer scale)
        for q in range(1, len(self.norms) + 1):
            n_in, n_out, n_mix, n_ls = _names(res, q)
            if res.connections:
                c = (f32(n_in, (S,)), f32(n_out, (S,)), f32(n_mix, (S, S)))
            else:
                one = torch.ones((1,), dtype=torch.float32, device=device)
                c = (None, one, one.view(1, 1))
            self.coef.append(c + (f32(n_ls, (res.hidden,)) if res.layer_scale else None,))

    def parts(self):
        return [self.mixer, self.ffn, *self.norms, getattr(self.mixer, "position", None)]

    # ---- the model's two ends ---------------------------------------------------------------------
    def enter(self, ctx, rows: torch.Tensor) -> torch.Tensor:
        """The embedding's rows -> the streams."""
        return ops.streams_open(rows, self.res.streams)

    def leave(self, ctx, x: torch.Tensor, pending, rows: torch.Tensor, norm) -> torch.Tensor:
        """The final norm of the sum of the streams at the wanted rows (`pending` is in already)."""
        if norm is None:
            return ops.streams_step(x, rows=rows, h_dtype=self.dtype)
        if getattr(norm, "add_one", False):
            raise SpecError("streams: the final norm must be a plain RMS norm")
        return ops.streams_step(x, rows=rows, norm_weight=norm.weight, eps=norm.eps, h_dtype=self.dtype)

    # ---- a layer ------------------------------------------------------------------------------------
    @staticmethod
    def _add(x, y, coef, read=None, norm=None, dtype=None):
        """Adds sub-layer output `y` (rows, or a feed-forward's rows a chosen expert with their weights) into the
        streams and, with `norm`, returns the next sub-layer's input."""
        _, out, mix, ls = coef
        weights = None
        if hasattr(y, "rows") and hasattr(y, "weights"):
            y, weights = y.rows, y.weights
        elif hasattr(y, "materialize"):
            y = y.materialize()
        kw = dict(norm_weight=norm.weight, eps=norm.eps, h_dtype=dtype, read=read) if norm is not None else {}
        return ops.streams_step(x, y=y, y_weights=weights, scale=ls, mix=mix, out=out, **kw)

    def forward(self, ctx, x: torch.Tensor, pending, cache, next_norm=None) -> Tuple[torch.Tensor, object]:
        if x.dim() != 3 or x.dtype != torch.float32 or x.shape[1] != self.res.streams:
            raise SpecError(f"streams: the block takes 32-bit streams [tokens, {self.res.streams}, width], got {tuple(x.shape)} {x.dtype}")
        ctx.stream = ctx.stream_norm = None
        ctx.partial_sums = False
        # every block of this arrangement leaves the streams complete: nothing is pending between blocks
        h = ops.streams_step(x, read=self.coef[0][0], norm_weight=self.norms[0].weight, eps=self.norms[0].eps, h_dtype=self.dtype)
        a = self.mixer.forward(ctx, h, cache)
        if self.ffn is None:
            self._add(x, a, self.coef[0])
            return x, None
        h2 = self._add(x, a, self.coef[0], read=self.coef[1][0], norm=self.norms[1], dtype=self.dtype)
        self._add(x, self.ffn.forward(ctx, h2), self.coef[1])
        return x, None
