"""The real-gated linear recurrent unit behind a short causal convolution, beside a GELU branch (the recurrent
block of De et al., "Griffin: Mixing Gated Linear Recurrences with Local Attention for Efficient Language Models"):

    y = gelu_tanh(W_y h + b_y);   u = conv(W_x h + b_x)            (a convolution a channel, zeros before the start)
    r = sigmoid(A_b u_b + a_b),   i = sigmoid(I_b u_b + i_b)       (block-diagonal: part b of u through its own matrix)
    a = exp(-decay * r * softplus(lam));   S <- a S + sqrt(1 - a^2) * i * u;   out = W_o (S * y)

A request keeps the state S and the convolution's last `conv - 1` inputs, both in 32-bit, in its row of a
fixed-size state array; gates, decays and the recurrence are 32-bit.
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import GatedRecurrenceSpec, SpecError
from ..weights.loader import TensorSpec
from .base import FixedState, Mixer, register_mixer
from .linear import Linear, to_compute


@register_mixer("rglru")
class GatedRecurrence(Mixer):
    graph_safe = True
    CHUNKED_FROM = 64              # steps whose longest portion has more tokens walk it in chunks side by side

    @classmethod
    def tensors(cls, spec: GatedRecurrenceSpec) -> Dict[str, TensorSpec]:
        w, b = spec.width, spec.blocks
        bw = w // b
        return {
            "y": TensorSpec((w, spec.hidden)), "y.b": TensorSpec((w,)),
            "x": TensorSpec((w, spec.hidden)), "x.b": TensorSpec((w,)),
            "conv": TensorSpec((w, spec.conv)), "conv.b": TensorSpec((w,)),
            "ra": TensorSpec((b, bw, bw)), "ra.b": TensorSpec((b, bw)),
            "ri": TensorSpec((b, bw, bw)), "ri.b": TensorSpec((b, bw)),
            "lam": TensorSpec((w,)),
            "o": TensorSpec((spec.hidden, w)),
        }

    @classmethod
    def cache_need(cls, spec: GatedRecurrenceSpec):
        # row 0: the recurrent state; rows 1..conv-1: the convolution's last inputs, oldest first
        return FixedState((spec.conv, spec.width), torch.float32)

    def __init__(self, spec: GatedRecurrenceSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        if spec.width % spec.blocks or spec.conv < 1:
            raise SpecError(f"rglru: width {spec.width} in {spec.blocks} blocks, {spec.conv} taps")
        self.spec = spec
        self.proj = Linear([tensors["y"], tensors["x"]], dtype, device, [tensors["y.b"], tensors["x.b"]])
        self.taps = to_compute(tensors["conv"], dtype, device).t().contiguous()          # [taps, width]: the kernels read tap by tap
        self.conv_bias = to_compute(tensors["conv.b"], dtype, device)
        # a block's two gate matrices one above the other: [blocks, 2 bw, bw]
        self.gates = torch.cat([to_compute(tensors["ra"], dtype, device), to_compute(tensors["ri"], dtype, device)], dim=1).contiguous()
        self.bias_r = to_compute(tensors["ra.b"], dtype, device).reshape(-1)
        self.bias_i = to_compute(tensors["ri.b"], dtype, device).reshape(-1)
        self.lam = to_compute(tensors["lam"], dtype, device)
        self.o = Linear([tensors["o"]], dtype, device)

    def forward(self, ctx, h, cache):
        s = self.spec
        w, bw = s.width, s.width // s.blocks
        proj = self.proj(h)                                      # [n, gelu branch | convolution's input]
        lo = proj.dtype == torch.bfloat16               # the gates' products take u in the projections' precision
        u = ops.conv_step(proj, w, w, self.taps, self.conv_bias, cache.state, ctx.token_seq, ctx.cu_tokens, ctx.state_slots,
                          rounded=lo)
        u, u_in = u if lo else (u, u)
        z = ops.head_product(u_in, self.gates, out_dtype=torch.float32)               # [n, blocks * 2 bw]
        mixed = ops.rglru_scan(u, z, proj, branch_off=0, x_off=w, bias_r=self.bias_r, bias_i=self.bias_i, lam=self.lam,
                               state=cache.state, cu_tokens=ctx.cu_tokens, state_slots=ctx.state_slots, block_width=bw,
                               decay=s.decay, chunked=ctx.max_q_len > self.CHUNKED_FROM)
        return self.o(mixed)
