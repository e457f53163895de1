"""Mixers that carry a matrix of fixed size a head from token to token instead of a cache that grows:

    S_t = a_t S_(t-1) + b_t k_t v_t^T,      o_t = S_t^T q_t

with a decay a_t and an input scale b_t that are scalars a (token, head).  "retention" has a constant decay a head;
"mlstm" (the matrix memory of the xLSTM, Beck et al., "xLSTM: Extended Long Short-Term Memory") has exponential gates
under a running maximum and a normaliser; "mamba2" (Dao and Gu, "Transformers are SSMs") is a selective state space behind
a short convolution.  All three run on the same recurrence kernel (`ops.linear_scan`) and the same closing kernel
(`ops.group_norm_gate`: a norm a group of features and a gate); their gates have kernels of their own.  "side_by_side"
runs two mixers on the same input and hands both outputs, with their weights, to the kernel that adds them to the stream.

A request keeps its matrices (and the running maxima, or the convolution's last inputs) in its row of a fixed-size
32-bit state array; states, decays, gates, step sizes and the norms are 32-bit whatever the products' precision.
"""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import MatrixMemorySpec, RetentionSpec, SideBySideSpec, SpecError, StateSpaceSpec
from ..weights.loader import TensorSpec
from .base import FixedState, Mixer, PagedAndState, PagedKV, part_class, register_mixer
from .block import sub_tensors
from .linear import Linear, to_compute


def _f32(t: torch.Tensor, device) -> torch.Tensor:
    return t.to(device=device, dtype=torch.float32).reshape(-1).contiguous()


def _check_dim(kind: str, dim: int) -> None:
    if not (1 <= dim <= ops.state.SCAN_MAX_DIM):
        raise SpecError(f"{kind}: a key size of {dim} is outside 1..{ops.state.SCAN_MAX_DIM}, the range of the recurrence kernel")


@register_mixer("retention")
class Retention(Mixer):
    graph_safe = True

    @classmethod
    def tensors(cls, spec: RetentionSpec) -> Dict[str, TensorSpec]:
        qk, vv = spec.n_heads * spec.head_dim, spec.n_heads * spec.v_dim
        return {"q": TensorSpec((qk, spec.hidden)), "k": TensorSpec((qk, spec.hidden)), "v": TensorSpec((vv, spec.hidden)),
                "g": TensorSpec((vv, spec.hidden)), "o": TensorSpec((spec.hidden, vv))}

    @classmethod
    def cache_need(cls, spec: RetentionSpec):
        return FixedState((spec.n_heads * spec.v_dim * spec.head_dim,), torch.float32)

    def __init__(self, spec: RetentionSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        _check_dim("retention", spec.head_dim)
        if len(spec.decay) != spec.n_heads or any(not (0.0 <= d <= 1.0) for d in spec.decay):
            raise SpecError(f"retention: one decay in 0..1 for each of the {spec.n_heads} heads, got {list(spec.decay)}")
        self.spec = spec
        self.proj = Linear([tensors["q"], tensors["k"], tensors["v"], tensors["g"]], dtype, device)
        self.o = Linear([tensors["o"]], dtype, device)
        self.decay = torch.tensor([float(d) for d in spec.decay], dtype=torch.float32, device=device)

    def forward(self, ctx, h, cache):
        s = self.spec
        qk, vv = s.n_heads * s.head_dim, s.n_heads * s.v_dim
        proj = self.proj(h)                                   # [n, q | k | v | g]
        o = ops.linear_scan(q=proj, q_off=0, q_heads=s.n_heads, k=proj, k_off=qk, k_heads=s.n_heads, v=proj, v_off=2 * qk,
                            heads=s.n_heads, dim=s.head_dim, vdim=s.v_dim, state=cache.state, s_off=0,
                            cu_tokens=ctx.cu_tokens, state_slots=ctx.state_slots, decay=self.decay, max_q_len=ctx.max_q_len,
                            k_scale=s.head_dim ** -0.5)
        y = ops.group_norm_gate(o, group=s.v_dim, head=s.v_dim, eps=s.norm_eps, out_dtype=proj.dtype, gate=proj,
                                gate_off=2 * qk + vv, act=ops.state.ACT_SILU)
        return self.o(y)


@register_mixer("mlstm")
class MatrixMemory(Mixer):
    graph_safe = True

    @classmethod
    def tensors(cls, spec: MatrixMemorySpec) -> Dict[str, TensorSpec]:
        qk, vv, H = spec.n_heads * spec.head_dim, spec.n_heads * spec.v_dim, spec.n_heads
        return {"q": TensorSpec((qk, spec.hidden)), "k": TensorSpec((qk, spec.hidden)), "v": TensorSpec((vv, spec.hidden)),
                "g": TensorSpec((vv, spec.hidden)), "o": TensorSpec((spec.hidden, vv)), "norm": TensorSpec((vv,), "norm"),
                "i": TensorSpec((H, spec.hidden)), "i.b": TensorSpec((H,)), "f": TensorSpec((H, spec.hidden)),
                "f.b": TensorSpec((H,))}

    @classmethod
    def cache_need(cls, spec: MatrixMemorySpec):
        # the matrices with the normaliser's column, [heads][v_dim + 1][dim], then the running maxima [heads]
        return FixedState((spec.n_heads * (spec.v_dim + 1) * spec.head_dim + spec.n_heads,), torch.float32)

    def __init__(self, spec: MatrixMemorySpec, tensors: Dict[str, torch.Tensor], dtype, device):
        _check_dim("mlstm", spec.head_dim)
        if not spec.gate_cap > 0.0:
            raise SpecError(f"mlstm: the gates' cap must be positive, got {spec.gate_cap}")
        self.spec = spec
        self.proj = Linear([tensors[n] for n in ("q", "k", "v", "g", "i", "f")], dtype, device)
        self.o = Linear([tensors["o"]], dtype, device)
        self.bias_i, self.bias_f = _f32(tensors["i.b"], device), _f32(tensors["f.b"], device)
        self.norm = _f32(tensors["norm"], device)

    def forward(self, ctx, h, cache):
        s = self.spec
        qk, vv, H = s.n_heads * s.head_dim, s.n_heads * s.v_dim, s.n_heads
        proj = self.proj(h)                                   # [n, q | k | v | g | i | f]
        m_off = H * (s.v_dim + 1) * s.head_dim
        log_a, b, floor = ops.exp_gates(proj, 2 * qk + 2 * vv, 2 * qk + 2 * vv + H, self.bias_i, self.bias_f, s.gate_cap,
                                        cache.state, m_off, ctx.cu_tokens, ctx.state_slots, max_q_len=ctx.max_q_len)
        o, den = ops.linear_scan(q=proj, q_off=0, q_heads=H, k=proj, k_off=qk, k_heads=H, v=proj, v_off=2 * qk, heads=H,
                                 dim=s.head_dim, vdim=s.v_dim, state=cache.state, s_off=0, cu_tokens=ctx.cu_tokens,
                                 state_slots=ctx.state_slots, log_a=log_a, b=b, q_scale=s.head_dim ** -0.5, normaliser=True,
                                 max_q_len=ctx.max_q_len)
        y = ops.group_norm_gate(o, group=s.v_dim, head=s.v_dim, eps=s.norm_eps, out_dtype=proj.dtype, weight=self.norm,
                                gate=proj, gate_off=2 * qk + vv, act=ops.state.ACT_SIGMOID, den=den, floor=floor)
        return self.o(y)


@register_mixer("mamba2")
class StateSpace(Mixer):
    graph_safe = True

    @classmethod
    def _sizes(cls, spec: StateSpaceSpec):
        inner, bc = spec.n_heads * spec.v_dim, spec.groups * spec.state
        return inner, bc, inner + 2 * bc                       # inner, one of B and C, the convolution's channels

    @classmethod
    def tensors(cls, spec: StateSpaceSpec) -> Dict[str, TensorSpec]:
        inner, bc, channels = cls._sizes(spec)
        H = spec.n_heads
        return {"in": TensorSpec((2 * inner + 2 * bc + H, spec.hidden)), "conv": TensorSpec((channels, spec.conv)),
                "conv.b": TensorSpec((channels,)), "dt_bias": TensorSpec((H,)), "A_log": TensorSpec((H,)),
                "D": TensorSpec((H,), "norm"), "norm": TensorSpec((inner,), "norm"), "o": TensorSpec((spec.hidden, inner))}

    @classmethod
    def cache_need(cls, spec: StateSpaceSpec):
        inner, _, channels = cls._sizes(spec)
        # the matrices [heads][v_dim][state], then the convolution's last inputs [conv - 1][channels]
        return FixedState((inner * spec.state + (spec.conv - 1) * channels,), torch.float32)

    def __init__(self, spec: StateSpaceSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        _check_dim("mamba2", spec.state)
        inner, _, _ = self._sizes(spec)
        if spec.n_heads % spec.groups or inner % spec.norm_groups or spec.conv < 1:
            raise SpecError(f"mamba2: {spec.n_heads} heads in {spec.groups} groups, {inner} features in {spec.norm_groups} "
                            f"norm groups, {spec.conv} taps")
        self.spec = spec
        self.proj = Linear([tensors["in"]], dtype, device)
        self.o = Linear([tensors["o"]], dtype, device)
        self.taps = to_compute(tensors["conv"], dtype, device).t().contiguous()         # [taps, channels]: the kernel reads tap by tap
        self.conv_bias = to_compute(tensors["conv.b"], dtype, device)
        self.dt_bias, self.a_log = _f32(tensors["dt_bias"], device), _f32(tensors["A_log"], device)
        self.skip, self.norm = _f32(tensors["D"], device), _f32(tensors["norm"], device)

    def forward(self, ctx, h, cache):
        s = self.spec
        inner, bc, channels = self._sizes(s)
        proj = self.proj(h)                                   # [n, z | x | B | C | dt]
        xbc = ops.conv_act_step(proj, inner, channels, self.taps, self.conv_bias, cache.state, inner * s.state,
                                ctx.token_seq, ctx.cu_tokens, ctx.state_slots, act=ops.state.ACT_SILU)
        log_a, b = ops.step_gates(proj, 2 * inner + 2 * bc, self.dt_bias, self.a_log)
        y = ops.linear_scan(q=xbc, q_off=inner + bc, q_heads=s.groups, k=xbc, k_off=inner, k_heads=s.groups, v=xbc, v_off=0,
                            heads=s.n_heads, dim=s.state, vdim=s.v_dim, state=cache.state, s_off=0, cu_tokens=ctx.cu_tokens,
                            state_slots=ctx.state_slots, log_a=log_a, b=b, skip=self.skip, max_q_len=ctx.max_q_len)
        y = ops.group_norm_gate(y, group=inner // s.norm_groups, head=s.v_dim, eps=s.norm_eps, out_dtype=proj.dtype,
                                weight=self.norm, gate=proj, gate_off=0, act=ops.state.ACT_SILU, gate_first=True)
        return self.o(y)


@register_mixer("side_by_side")
class SideBySide(Mixer):
    """Two mixers on the same input.  One of them may keep pages and the other a state (`PagedAndState`); two needs of
    one sort are refused."""

    @classmethod
    def tensors(cls, spec: SideBySideSpec) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for side, prefix in ((spec.left, spec.left_prefix), (spec.right, spec.right_prefix)):
            for local, ts in part_class("mixer", side).tensors(side).items():
                out[prefix + local] = ts
        return out

    @classmethod
    def cache_need(cls, spec: SideBySideSpec):
        needs = [part_class("mixer", side).cache_need(side) for side in (spec.left, spec.right)]
        needs = [n for n in needs if n is not None]
        if len(needs) <= 1:
            return needs[0] if needs else None
        paged = [n for n in needs if isinstance(n, PagedKV)]
        state = [n for n in needs if isinstance(n, FixedState)]
        if len(paged) != 1 or len(state) != 1:
            raise SpecError("side_by_side: of two mixers that keep something, one keeps pages and the other a state")
        return PagedAndState(paged[0], state[0])

    def __init__(self, spec: SideBySideSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec = spec
        self.left = part_class("mixer", spec.left)(spec.left, sub_tensors(tensors, spec.left_prefix), dtype, device)
        self.right = part_class("mixer", spec.right)(spec.right, sub_tensors(tensors, spec.right_prefix), dtype, device)
        self.position = getattr(self.left, "position", None) or getattr(self.right, "position", None)

    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.left, "graph_safe", False) and getattr(self.right, "graph_safe", False))

    def parts(self):
        return [self.left, self.right]

    def load_notes(self, page_size: int):
        return [n for side in (self.left, self.right) if hasattr(side, "load_notes") for n in side.load_notes(page_size)]

    def forward(self, ctx, h, cache):
        left, right = self.left.forward(ctx, h, cache), self.right.forward(ctx, h, cache)
        if hasattr(left, "materialize"):
            left = left.materialize()
        if hasattr(right, "materialize"):
            right = right.materialize()
        return ops.state.WeightedPair(left, self.spec.left_scale, right, self.spec.right_scale)
