"""A plain, slow implementation of the Buketar decoder: whole sequences, no cache, no paging, no
batching, one function per mechanism, plain torch arithmetic on the CPU in one precision (float64
by default).  It shares no code with `inferrs_amd`: a model is a config dictionary (the keys of
config.json) and a dictionary of tensors by their names in the file.

The design in short.  A token's row is copied into `streams` residual streams.  Every layer has a
mixer (latent attention, or a gated linear recurrence with a short convolution in front) and an
optional feed-forward of routed experts.  A sub-layer reads a weighted sum of the streams through
an RMS norm, its output is scaled per feature, and the streams are remixed by a small matrix with
the output added to each of them with a weight of its own.  A range of layers may run several
times in a row.  The logits are capped by a tanh.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch

T = Dict[str, torch.Tensor]


# ---- small pieces ---------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


# ---- rotary positions with the YaRN law ---------------------------------------------------------

def rotary_frequencies(rot: dict, dtype=torch.float64) -> (torch.Tensor, float):
    """(frequency of every pair, factor on cos and sin).  Pair i of `dims` features turns by
    base^(-2i/dims) a position; under a scaling law the low frequencies are divided by `factor`,
    the high ones kept, with a linear ramp between the pairs that make `fast` and `slow` turns
    over `original` positions."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=dtype)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def pair_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(pair_of(float(sc["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=dtype)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [..., tokens, n]: the first rot.dims features turn, feature i paired with i + dims/2."""
    dims = int(rot["dims"])
    half = dims // 2
    f, m = rotary_frequencies(rot, x.dtype)
    ang = positions.to(x.dtype)[:, None] * f[None, :]
    c, s = torch.cos(ang) * m, torch.sin(ang) * m
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


# ---- mixer: latent attention ----------------------------------------------------------------------

def latent_attention(h: torch.Tensor, w: T, m: dict, eps: float, positions: torch.Tensor) -> torch.Tensor:
    """Keys and values of all heads are formed from one low-rank row a token (`kv_rank` wide, RMS
    normed) plus one rotated key part shared by the heads; the joined heads are gated by a sigmoid
    of a projection of the same input."""
    n = h.shape[0]
    H, d, r, dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    q = (h @ w["q"].T).view(n, H, d + r).transpose(0, 1)                # [H, n, d + r]
    down = h @ w["dkv"].T
    c = rms_norm(down[:, :rank], w["dkv.norm"], eps)
    k_rot = rotate(down[:, rank:], positions, m["rot"])                   # [n, r], one for all heads
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], positions, m["rot"])
    k_plain = (c @ w["uk"].T).view(n, H, d).transpose(0, 1)
    v = (c @ w["uv"].T).view(n, H, dv).transpose(0, 1)
    scores = (q_plain @ k_plain.transpose(1, 2) + q_rot @ k_rot.T[None]) * float(m["scale"])
    visible = positions[None, :] <= positions[:, None]
    scores = scores.masked_fill(~visible[None], float("-inf"))
    p = torch.softmax(scores, dim=-1)
    joined = (p @ v).transpose(0, 1).reshape(n, H * dv)
    return (joined * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


# ---- mixer: gated linear recurrence -----------------------------------------------------------------

def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """Per channel; the last tap meets the current token, zeros stand before the first token."""
    n, k = x.shape[0], taps.shape[1]
    padded = torch.cat([x.new_zeros(k - 1, x.shape[1]), x], dim=0)
    out = bias.expand(n, -1).clone()
    for j in range(k):
        out = out + padded[j:j + n] * taps[:, j]
    return out


def block_gate(u: torch.Tensor, mats: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """sigmoid of a block-diagonal product: part b of u through mats[b] ([out, in])."""
    n, blocks = u.shape[0], mats.shape[0]
    parts = u.view(n, blocks, -1)
    z = torch.einsum("nbi,boi->nbo", parts, mats) + bias
    return torch.sigmoid(z).reshape(n, -1)


def rglru(h: torch.Tensor, w: T, m: dict) -> torch.Tensor:
    y = gelu_tanh(h @ w["y"].T + w["y.b"])
    u = causal_conv(h @ w["x"].T + w["x.b"], w["conv"], w["conv.b"])
    r = block_gate(u, w["ra"], w["ra.b"])
    i = block_gate(u, w["ri"], w["ri.b"])
    log_a = -8.0 * r * softplus(w["lam"])
    a = torch.exp(log_a)
    drive = torch.sqrt(1.0 - a * a) * i * u
    state = torch.zeros_like(u[0])
    rows = []
    for t in range(u.shape[0]):
        state = a[t] * state + drive[t]
        rows.append(state)
    return (torch.stack(rows) * y) @ w["o"].T


# ---- feed-forward: routed experts ------------------------------------------------------------------

def expert(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float) -> torch.Tensor:
    g = (h @ gate.T).clamp(max=limit)
    u = (h @ up.T).clamp(min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def routed_experts(h: torch.Tensor, w: T, f: dict) -> torch.Tensor:
    n_exp, top, scale = int(f["router"]["experts"]), int(f["router"]["top"]), float(f["router"]["scale"])
    limit = float(f["expert"]["limit"])
    s = torch.sigmoid(h @ w["router"].T)
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        chosen = sorted(range(n_exp), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in chosen:
            out[t] += s[t, e] * scale * expert(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)[0]
    return out


# ---- the model ---------------------------------------------------------------------------------------

def sub(tensors: T, prefix: str) -> T:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def run_order(cfg: dict) -> List[int]:
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg: dict, tensors: T, tokens: Sequence[int], dtype=torch.float64, layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [tokens, vocab] of one sequence from its start.  `layers_out`: a list that receives the
    sum of the streams after every layer run."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = float(cfg["norm"]["eps"])
    positions = torch.arange(len(tokens))
    x = w["embed"][torch.tensor(list(tokens))]
    n_streams = cfg.get("streams")
    streams = [x.clone() for _ in range(int(n_streams))] if n_streams else [x]
    for li in run_order(cfg):
        layer, p = cfg["layers"][li], f"l{li}."
        for q, kind in ((1, "mixer"), (2, "mlp")):
            if kind == "mlp" and layer.get("mlp") is None:
                continue
            if n_streams:
                u = sum(w[f"{p}hc{q}.in"][s] * streams[s] for s in range(len(streams)))
            else:
                u = streams[0]
            h = rms_norm(u, w[f"{p}norm{q}"], eps)
            if kind == "mixer":
                mw = sub(w, p + "mix.")
                if layer["type"] == "latent_attention":
                    y = latent_attention(h, mw, layer["mixer"], eps, positions)
                elif layer["type"] == "rglru":
                    y = rglru(h, mw, layer["mixer"])
                else:
                    raise ValueError(layer["type"])
            else:
                y = routed_experts(h, sub(w, p + "mlp."), layer["mlp"])
            y = y * w[f"{p}ls{q}"]
            if n_streams:
                mix, out = w[f"{p}hc{q}.mix"], w[f"{p}hc{q}.out"]
                streams = [sum(mix[s, t] * streams[s] for s in range(len(streams))) + out[t] * y
                           for t in range(len(streams))]
            else:
                streams = [streams[0] + y]
        if layers_out is not None:
            layers_out.append(sum(streams))
    x = rms_norm(sum(streams), w["final.norm"], eps)
    logits = x @ w["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def load_folder(folder: str):
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for k in f.keys():
            tensors[k] = f.get_tensor(k)
    return cfg, tensors
