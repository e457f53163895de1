"""A plain, slow implementation of the Lofudra decoder: whole sequences, no cache, no paging, no
batching, one function per mechanism, plain torch arithmetic on the CPU in one precision (float64
by default).  It shares no code with `inferrs_amd`: a model is a config dictionary (the keys of
config.json) and a dictionary of tensors by their names in the file.

The design in short.  Every layer has a mixer and an optional dense feed-forward, each between a norm
in front and a norm behind: x += norm_b(part(norm_a(x))).  Three mixers: "parallel" (a sliding-window
softmax attention whose values are its un-normed, un-rotated keys and whose softmax has a sink of score
0, side by side with a retention of fixed decays, the two added with fixed weights), "mlstm" (the
matrix memory of the xLSTM with capped exponential gates and a running maximum) and "mamba2" (a
selective state space behind a short convolution).  A range of layers may run several times in a row;
before every pass a learned vector is added, and before every pass but the first the embedding's row
once more.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

T = Dict[str, torch.Tensor]


# ---- small pieces ---------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


def log_sigmoid(z: torch.Tensor) -> torch.Tensor:
    return -softplus(-z)


def dense_ff(h: torch.Tensor, w: T, p: str) -> torch.Tensor:
    """down(gelu(up h)), the exact GELU."""
    return gelu_erf(h @ w[p + "up"].T) @ w[p + "down"].T


# ---- the windowed attention with a sink; its values are its un-normed, un-rotated keys ----------------

def rotate_halves(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [tokens, heads, dim]: the first `dims` features of every head turn, feature i with i + dims/2."""
    if dims == 0:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    a = positions.to(x.dtype)[:, None, None] * f[None, None, :]
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def sink_window_attention(h: torch.Tensor, w: T, p: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    window, scale = int((m.get("mask") or {}).get("size", n + 1)), float(m["scale"])      # no mask: every earlier key
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(n, H, d)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(n, G, d)
    v = k                                             # (no value projection: the key rows themselves, ahead of norm and turn)
    pos = torch.arange(n)
    rot = m.get("rot") or {}
    q = rotate_halves(rms_norm(q, w[p + "q.norm"], eps), pos, float(rot.get("base", 1.0)), int(rot.get("dims", 0)))
    k = rotate_halves(rms_norm(k, w[p + "k.norm"], eps), pos, float(rot.get("base", 1.0)), int(rot.get("dims", 0)))
    out = torch.zeros(n, H, d, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * scale                     # [query, key]
        i, j = pos[:, None], pos[None, :]
        seen = (j <= i) & (i - j < window)
        e = torch.where(seen, torch.exp(s), torch.zeros_like(s))
        out[:, head] = (e / (1.0 + e.sum(dim=1, keepdim=True))) @ v[:, g]
    return out.reshape(n, H * d) @ w[p + "o"].T


# ---- retention -------------------------------------------------------------------------------------

def retention(h: torch.Tensor, w: T, p: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[p + "q"].T).view(n, H, d)
    k = (h @ w[p + "k"].T).view(n, H, d) * d ** -0.5
    v = (h @ w[p + "v"].T).view(n, H, dv)
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    for head in range(H):
        decay = float(m["decay"][head])
        S = torch.zeros(d, dv, dtype=h.dtype)
        for t in range(n):
            S = decay * S + torch.outer(k[t, head], v[t, head])
            out[t, head] = S.T @ q[t, head]
    out = rms_norm(out, None, eps).reshape(n, H * dv)
    return (out * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def parallel_mixer(h: torch.Tensor, w: T, p: str, m: dict, eps: float) -> torch.Tensor:
    left = sink_window_attention(h, w, p + "left.", m["left"], eps)
    right = retention(h, w, p + "right.", m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


# ---- the matrix memory with exponential gates ------------------------------------------------------

def mlstm(h: torch.Tensor, w: T, p: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, d, dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    q = (h @ w[p + "q"].T).view(n, H, d) * d ** -0.5
    k = (h @ w[p + "k"].T).view(n, H, d)
    v = (h @ w[p + "v"].T).view(n, H, dv)
    gi = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)                       # [n, H], a logarithm
    gf = log_sigmoid(cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    for head in range(H):
        S = torch.zeros(d, dv, dtype=h.dtype)
        norm = torch.zeros(d, dtype=h.dtype)
        top = torch.zeros((), dtype=h.dtype)               # the running maximum starts at 0
        for t in range(n):
            new_top = torch.maximum(gf[t, head] + top, gi[t, head])
            keep, take = torch.exp(gf[t, head] + top - new_top), torch.exp(gi[t, head] - new_top)
            S = keep * S + take * torch.outer(k[t, head], v[t, head])
            norm = keep * norm + take * k[t, head]
            top = new_top
            below = torch.maximum((norm @ q[t, head]).abs(), torch.exp(-top)) + 1e-6
            out[t, head] = (S.T @ q[t, head]) / below
    out = rms_norm(out, None, eps).reshape(n, H * dv) * w[p + "norm"]
    return (out * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


# ---- the selective state space ---------------------------------------------------------------------

def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x [tokens, channels], taps [channels, taps]: the last tap meets the current token; ahead of a sequence's first token there is nothing but zeros."""
    n, k = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros(k - 1, x.shape[1], dtype=x.dtype), x], dim=0)
    out = bias.expand(n, -1).clone()
    for j in range(k):
        out = out + padded[j:j + n] * taps[:, j]
    return out


def mamba2(h: torch.Tensor, w: T, p: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, dv, N, G, parts = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["norm_groups"])
    inner = H * dv
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(n, H, dv)
    B = xbc[:, inner:inner + G * N].view(n, G, N)
    C = xbc[:, inner + G * N:].view(n, G, N)
    dt = softplus(dt + w[p + "dt_bias"])                           # [n, H]
    rate = torch.exp(w[p + "A_log"])
    y = torch.zeros(n, H, dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(N, dv, dtype=h.dtype)
        for t in range(n):
            S = torch.exp(-rate[head] * dt[t, head]) * S + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S.T @ C[t, g] + w[p + "D"][head] * x[t, head]
    y = y.reshape(n, inner) * silu(z)                               # gated first, normed second
    y = rms_norm(y.view(n, parts, inner // parts), None, eps).reshape(n, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


MIXERS = {"parallel": parallel_mixer, "mlstm": mlstm, "mamba2": mamba2}


# ---- the model ----------------------------------------------------------------------------------------

def layer_forward(x: torch.Tensor, w: T, i: int, layer: dict, eps: float) -> torch.Tensor:
    p = f"l{i}."
    a = MIXERS[layer["type"]](rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], eps)
    x = x + rms_norm(a, w[p + "norm1b"], eps)
    if layer.get("mlp") is not None:
        f = dense_ff(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.")
        x = x + rms_norm(f, w[p + "norm2b"], eps)
    return x


def passes(cfg: dict) -> List[Sequence[int]]:
    """The runs of layers; each entry (layers, pass number or None for layers outside the loop)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(list(range(n)), None)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    out = [(list(range(a)), None)] if a else []
    out += [(list(range(a, b)), t) for t in range(times)]
    if b < n:
        out.append((list(range(b, n)), None))
    return out


def forward(cfg: dict, weights: T, tokens: Sequence[int], dtype=torch.float64, trace: Optional[list] = None) -> torch.Tensor:
    """Logits [tokens, vocab] of one whole sequence; `trace` collects the stream after every layer run."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    first = w["embed"][torch.as_tensor(list(tokens), dtype=torch.long)]
    x = first
    for layers, t in passes(cfg):
        if t is not None:
            if t > 0:
                x = x + first
            x = x + w["loop.step"][t]
        for i in layers:
            x = layer_forward(x, w, i, cfg["layers"][i], eps)
            if trace is not None:
                trace.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T
