"""Python face of the kernels for a 32-bit stream between two norms a sub-layer (`csrc/sandwich.hip`) and for mixers
that carry a matrix state a head (`csrc/linear_state.hip`): retention, the matrix memory with exponential gates, the
selective state space.  Shape checks on the host, then one C call a kernel; no other implementation stands behind them.

A request's state is its row of a 32-bit array [slots, row_floats]; every call names the offset of its part of the row.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import KernelError, _DT, _check, _dev, _dt, _f32, _i32, _p, _stream, library

ACT_SILU, ACT_GELU_TANH, ACT_GELU, ACT_SIGMOID = 1, 2, 3, 4
SCAN_MAX_DIM = 512            # rows of a head's matrix that the recurrence kernel takes
SCAN_CHUNK = 64               # tokens of a chunk when long portions run in chunks side by side
SCAN_CHUNKS_FROM = 128        # steps whose longest portion has more tokens than this run in chunks
SCAN_WORKSPACE_FLOATS = 1 << 28   # the chunks' matrices take no more than this (1 GiB): longer chunks beyond


# ---- the stream ---------------------------------------------------------------------------------------------------

def sandwich_step(x: torch.Tensor, *, y: Optional[torch.Tensor] = None, y_scale: float = 1.0,
                  y2: Optional[torch.Tensor] = None, y2_scale: float = 1.0, post_weight: Optional[torch.Tensor] = None,
                  enter_rows: Optional[torch.Tensor] = None, enter_vector: Optional[torch.Tensor] = None,
                  pre_weight: Optional[torch.Tensor] = None, post_eps: float = 0.0, eps: float = 0.0,
                  h_dtype: Optional[torch.dtype] = None, rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """What stands between two sub-layers around a 32-bit stream x [n, width] (changed in place):

        x += rmsnorm(y_scale * y + y2_scale * y2) * post_weight (with `post_eps`);  x += enter_rows + enter_vector;
        returns rmsnorm(x) * pre_weight (with `eps`) in `h_dtype` (None: nothing is returned).

    Every half may be absent.  `rows` (int32): only these rows are read, the stream is left as it is and the result has
    one row for each of them."""
    _dev(x, y, y2, post_weight, enter_rows, enter_vector, pre_weight, rows)
    _f32(x, "the stream"); _f32(post_weight, "post weight"); _f32(pre_weight, "pre weight"); _f32(enter_vector, "enter vector")
    n, W = x.shape
    for t, name in ((y, "y"), (y2, "y2"), (enter_rows, "enter_rows")):
        if t is not None and tuple(t.shape) != (n, W):
            raise KernelError(f"sandwich_step: {name} {tuple(t.shape)} does not fit the stream [{n}, {W}]")
    given = [t for t in (y, y2, enter_rows) if t is not None]
    if any(t.dtype != given[0].dtype for t in given):
        raise KernelError("sandwich_step: the outputs and the entering rows share one precision")
    if y2 is not None and y is None:
        raise KernelError("sandwich_step: a second output goes with a first")
    if y is not None and (post_weight is None or post_weight.numel() != W):
        raise KernelError("sandwich_step: an output to add needs the weight of the norm behind it")
    for t, name in ((pre_weight, "pre weight"), (enter_vector, "enter vector")):
        if t is not None and t.numel() != W:
            raise KernelError(f"sandwich_step: {name} has {t.numel()} entries, the stream is {W} wide")
    count = n
    if rows is not None:
        _i32(rows, "rows")
        count = rows.numel()
    h = torch.empty((count, W), dtype=h_dtype, device=x.device) if h_dtype is not None else None
    y_dt = _dt(given[0]) if given else 0
    _check(library().ia_sandwich_step(
        _p(x), _p(y), ctypes.c_float(y_scale), _p(y2), ctypes.c_float(y2_scale), _p(post_weight), _p(enter_rows),
        _p(enter_vector), _p(pre_weight), ctypes.c_float(post_eps), ctypes.c_float(eps), _p(h), _p(rows), count, W, y_dt,
        _DT[h_dtype] if h_dtype is not None else 0, _stream()))
    return h


def activation(x: torch.Tensor, act: int) -> torch.Tensor:
    """act over every element of x, in place: ACT_SILU, ACT_GELU_TANH, ACT_GELU (the exact one)."""
    _dev(x)
    _check(library().ia_activation(_p(x), ctypes.c_longlong(x.numel()), act, _dt(x), _stream()))
    return x


# ---- mixers with a matrix state -----------------------------------------------------------------------------------

def _state(state: torch.Tensor) -> int:
    _f32(state, "state")
    if state.dim() != 2:
        raise KernelError(f"the state array is [slots, floats a request], got {tuple(state.shape)}")
    return state.shape[1]


def conv_act_step(x: torch.Tensor, x_off: int, channels: int, taps: torch.Tensor, bias: Optional[torch.Tensor],
                  state: torch.Tensor, tail_off: int, token_seq: torch.Tensor, cu_tokens: torch.Tensor,
                  state_slots: torch.Tensor, act: int = ACT_SILU) -> torch.Tensor:
    """A causal convolution a channel over x[:, x_off : x_off + channels] with its activation, in the precision of x;
    `taps` [k, channels] (the last meets the current token); the inputs before a request's portion come from the
    [k - 1, channels] floats at `tail_off` of its state row, which then take the portion's last inputs."""
    _dev(x, taps, bias, state, token_seq, cu_tokens, state_slots)
    _i32(token_seq, "token_seq"); _i32(cu_tokens, "cu_tokens"); _i32(state_slots, "state_slots")
    row = _state(state)
    n, k = x.shape[0], taps.shape[0]
    if tuple(taps.shape) != (k, channels) or taps.dtype != x.dtype or (bias is not None and (bias.numel() != channels or bias.dtype != x.dtype)):
        raise KernelError(f"conv_act_step: taps {tuple(taps.shape)} do not fit {channels} channels in the precision of x")
    out = torch.empty((n, channels), dtype=x.dtype, device=x.device)
    _check(library().ia_conv_act_step(_p(out), _p(x), _p(taps), _p(bias), _p(state), row, tail_off, _p(token_seq),
                                      _p(cu_tokens), _p(state_slots), n, state_slots.numel(), channels, k, x.shape[1], x_off,
                                      act, _dt(x), _stream()))
    return out


def exp_gates(proj: torch.Tensor, i_off: int, f_off: int, bias_i: torch.Tensor, bias_f: torch.Tensor, cap: float,
              state: torch.Tensor, m_off: int, cu_tokens: torch.Tensor, state_slots: torch.Tensor, max_q_len: int = 0
              ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Exponential gates under a running maximum: with i = cap tanh((proj_i + bias_i) / cap), f = logsigmoid(cap
    tanh((proj_f + bias_f) / cap)) and m_t = max(f + m_(t-1), i) (kept at `m_off` of the state row), returns 32-bit
    (log decay f + m_(t-1) - m_t, input scale exp(i - m_t), floor exp(-m_t)), each [n, heads].  `max_q_len`: an upper
    bound of the tokens a request brings (0: unknown, the step's tokens); long portions are walked by a block's threads side
    by side, which differs from the walk token by token by rounding."""
    _dev(proj, bias_i, bias_f, state, cu_tokens, state_slots)
    _f32(bias_i, "bias_i"); _f32(bias_f, "bias_f"); _i32(cu_tokens, "cu_tokens"); _i32(state_slots, "state_slots")
    row = _state(state)
    n, H = proj.shape[0], bias_i.numel()
    if bias_f.numel() != H:
        raise KernelError("exp_gates: one bias a head for each gate")
    outs = [torch.empty((n, H), dtype=torch.float32, device=proj.device) for _ in range(3)]
    _check(library().ia_exp_gates(_p(outs[0]), _p(outs[1]), _p(outs[2]), _p(state), row, m_off, _p(proj), proj.shape[1],
                                  i_off, f_off, _p(bias_i), _p(bias_f), ctypes.c_float(cap), _p(cu_tokens), _p(state_slots),
                                  H, state_slots.numel(), int(max_q_len) or n, _dt(proj), _stream()))
    return outs[0], outs[1], outs[2]


def step_gates(proj: torch.Tensor, dt_off: int, dt_bias: torch.Tensor, a_log: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Step sizes of a selective state space: dt = softplus(proj_dt + dt_bias); returns 32-bit (log decay
    -exp(a_log) dt, input scale dt), each [n, heads]."""
    _dev(proj, dt_bias, a_log); _f32(dt_bias, "dt_bias"); _f32(a_log, "a_log")
    n, H = proj.shape[0], dt_bias.numel()
    if a_log.numel() != H:
        raise KernelError("step_gates: one bias and one rate a head")
    log_a = torch.empty((n, H), dtype=torch.float32, device=proj.device)
    b = torch.empty_like(log_a)
    _check(library().ia_step_gates(_p(log_a), _p(b), _p(proj), proj.shape[1], dt_off, _p(dt_bias), _p(a_log), n, H,
                                   _dt(proj), _stream()))
    return log_a, b


def linear_scan(*, q: torch.Tensor, q_off: int, q_heads: int, k: torch.Tensor, k_off: int, k_heads: int,
                v: torch.Tensor, v_off: int, heads: int, dim: int, vdim: int, state: torch.Tensor, s_off: int,
                cu_tokens: torch.Tensor, state_slots: torch.Tensor, log_a: Optional[torch.Tensor] = None,
                decay: Optional[torch.Tensor] = None, b: Optional[torch.Tensor] = None,
                skip: Optional[torch.Tensor] = None, q_scale: float = 1.0, k_scale: float = 1.0,
                normaliser: bool = False, max_q_len: int = 0, chunk: Optional[int] = None):
    """The recurrence S <- a S + b k v^T, o = S^T q (+ skip v) over each request's tokens, from and into the
    [heads, vdim (+ 1), dim] floats at `s_off` of its state row.  q, k, v are 2-D rows of one precision; head h reads
    q[:, q_off + (h // (heads / q_heads)) * dim ...], likewise k, and v[:, v_off + h * vdim ...].  The decay is `log_a`
    [n, heads] (logarithms, a (token, head)) or `decay` [heads] (constants); `b` [n, heads] or 1.  `normaliser`: S has
    one more column whose value is always 1; returns (o, that column's output [n, heads]).  o is 32-bit [n, heads * vdim].
    `max_q_len`: an upper bound of the tokens a request brings (0: unknown, the step's tokens).  `chunk`: 0 walks every
    request's tokens in order; a number cuts portions into chunks of that many tokens that run side by side (three
    kernels: each chunk from nothing, the chunks' matrices in order, what each chunk's start contributes; for keys of
    up to 128 entries and chunks of up to 64 tokens the first and the third are products on the matrix cores in true
    32-bit), which differs from the walk by rounding; None: chunks of `SCAN_CHUNK` for steps with a portion of more than `SCAN_CHUNKS_FROM` tokens."""
    _dev(q, k, v, state, cu_tokens, state_slots, log_a, decay, b, skip)
    _f32(log_a, "log_a"); _f32(decay, "decay"); _f32(b, "b"); _f32(skip, "skip")
    _i32(cu_tokens, "cu_tokens"); _i32(state_slots, "state_slots")
    row = _state(state)
    n = q.shape[0]
    if q.dim() != 2 or k.dim() != 2 or v.dim() != 2 or k.shape[0] != n or v.shape[0] != n or not (q.dtype == k.dtype == v.dtype):
        raise KernelError("linear_scan: q, k and v are 2-D rows of one precision for the same tokens")
    if (log_a is None) == (decay is None):
        raise KernelError("linear_scan: either the decays' logarithms a token or the heads' constants")
    if log_a is not None and tuple(log_a.shape) != (n, heads) or decay is not None and decay.numel() != heads:
        raise KernelError("linear_scan: the decays do not fit the heads")
    if b is not None and tuple(b.shape) != (n, heads) or skip is not None and skip.numel() != heads:
        raise KernelError("linear_scan: input scales [n, heads], skips [heads]")
    if dim > SCAN_MAX_DIM:
        raise KernelError(f"linear_scan: a key size of {dim} is beyond {SCAN_MAX_DIM}")
    out = torch.empty((n, heads * vdim), dtype=torch.float32, device=q.device)
    den = torch.empty((n, heads), dtype=torch.float32, device=q.device) if normaliser else None
    a = log_a if log_a is not None else decay
    n_seqs = state_slots.numel()
    longest = int(max_q_len) or n
    if chunk is None:
        chunk = SCAN_CHUNK if longest > SCAN_CHUNKS_FROM else 0
        while chunk and n_seqs * -(-longest // chunk) * heads * (vdim + 1) * dim > SCAN_WORKSPACE_FLOATS:
            chunk *= 2
    lib = library()
    work = None
    if chunk:
        work = torch.empty((lib.ia_linear_scan_workspace(n_seqs, longest, chunk, heads, dim, vdim, int(normaliser)),),
                           dtype=torch.float32, device=q.device)
    _check(lib.ia_linear_scan(
        _p(out), _p(den), _p(state), row, s_off, _p(q), q.shape[1], q_off, q_heads, _p(k), k.shape[1], k_off, k_heads,
        _p(v), v.shape[1], v_off, _p(a), int(log_a is not None), _p(b), _p(skip), _p(cu_tokens), _p(state_slots),
        n_seqs, heads, dim, vdim, ctypes.c_float(q_scale), ctypes.c_float(k_scale), chunk, longest, _p(work), _dt(q), _stream()))
    return (out, den) if normaliser else out


def group_norm_gate(o: torch.Tensor, *, group: int, head: int, eps: float, out_dtype: torch.dtype,
                    weight: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, gate_off: int = 0,
                    act: int = ACT_SILU, gate_first: bool = False, den: Optional[torch.Tensor] = None,
                    floor: Optional[torch.Tensor] = None) -> torch.Tensor:
    """What follows a recurrence: o [n, inner] (32-bit) is divided by max(|den|, floor) + 1e-6 a (token, head of `head`
    features) when `den` is given, multiplied by act(gate[:, gate_off ...]) before (`gate_first`) or behind an RMS norm over
    groups of `group` neighbouring features with `weight`; returns [n, inner] in `out_dtype`."""
    _dev(o, weight, gate, den, floor)
    _f32(o, "o"); _f32(weight, "weight"); _f32(den, "den"); _f32(floor, "floor")
    n, inner = o.shape
    if inner % group or inner % head or (weight is not None and weight.numel() != inner):
        raise KernelError(f"group_norm_gate: {inner} features in groups of {group}, heads of {head}")
    if gate is not None and (gate.dim() != 2 or gate.shape[0] != n or gate.dtype != out_dtype):
        raise KernelError("group_norm_gate: the gate is 2-D rows in the precision of the result")
    if (den is None) != (floor is None) or (den is not None and (den.shape != floor.shape or den.numel() != n * (inner // head))):
        raise KernelError("group_norm_gate: a normaliser and its floor, one a (token, head)")
    out = torch.empty((n, inner), dtype=out_dtype, device=o.device)
    _check(library().ia_group_norm_gate(
        _p(out), _p(o), _p(den), _p(floor), head, _p(gate), gate.shape[1] if gate is not None else 0, gate_off, act,
        int(gate_first), _p(weight), ctypes.c_float(eps), n, inner, group, _DT[out_dtype], _stream()))
    return out


class WeightedPair:
    """The outputs of two mixers side by side that are still to be added: left_scale * left + right_scale * right
    (the kernel that takes them into the stream forms the sum in 32-bit)."""
    __slots__ = ("left", "left_scale", "right", "right_scale")

    def __init__(self, left: torch.Tensor, left_scale: float, right: torch.Tensor, right_scale: float):
        self.left, self.left_scale, self.right, self.right_scale = left, float(left_scale), right, float(right_scale)
