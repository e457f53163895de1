"""Tiny Lofudra configurations that differ in every size and option, and random weights for them.

The tensor list is written out here from the design (not asked of the package), so a part that expects another name
or shape fails to load.  Weights are drawn so that the mechanisms matter: matrices N(0, 1/in), retention decays and
state-space rates spread from forgetting at once to remembering for hundreds of tokens, gate biases that let the
matrix memory's running maximum move; `sharpen` multiplies the attention's query projection so that a query singles
out a few keys of its window against the sink, and a key that is lost, read from a wrong page or one place outside
the window changes the logits by far more than rounding."""
from __future__ import annotations

import json
import os
from typing import Dict

import torch


def left(heads, kv_heads, dim, scale, window=None, base=10000.0, turned=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
         "rot": {"base": base, "dims": dim if turned is None else turned}}
    if window is not None:
        m["mask"] = {"size": window}
    return m


def right(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def parallel(l, r, ls, rs):
    return {"type": "parallel", "mixer": {"left": l, "right": r, "left_scale": ls, "right_scale": rs}}


def mlstm(heads, dim, vdim, cap):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def mamba2(heads, vdim, state, groups, conv, norm_groups):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}}


def layer(mixer, ff):
    return dict(mixer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


# A: a looped pair, grouped keys, part of a head rotating, a window of 24 (a page and a half), a head size of 16 (matrix
# cores in bfloat16), value sizes other than key sizes in the recurrences, a layer without feed-forward.
CFG_A = {"architecture": "Lofudra", "vocab": 211, "width": 48, "norm": {"eps": 1e-5},
         "loop": {"start": 1, "stop": 3, "times": 2},
         "layers": [layer(mamba2(3, 8, 16, 1, 3, 3), 40),
                    layer(parallel(left(4, 2, 16, 0.3, window=24, base=1000.0, turned=8), right(2, 8, 24, [0.9, 0.995]), 0.7, 1.2), 40),
                    layer(mlstm(2, 24, 16, 10.0), 56),
                    layer(parallel(left(4, 2, 16, 0.3, window=24, base=1000.0, turned=8), right(2, 8, 24, [0.9, 0.995]), 0.7, 1.2), None)]}
# B: no loop; head size 64 (the fused decode kernel in bfloat16), as many key heads as query heads, a window of 100, one
# tap, as many groups as heads, one norm group, a retention head of a single decay near 1.
CFG_B = {"architecture": "Lofudra", "vocab": 97, "width": 64, "norm": {"eps": 1e-6},
         "layers": [layer(parallel(left(2, 2, 64, 0.125, window=100, base=500000.0), right(1, 16, 16, [0.999]), 1.0, 0.5), 72),
                    layer(mamba2(4, 16, 8, 4, 1, 1), 72),
                    layer(mlstm(1, 16, 32, 4.0), None)]}
# C: recurrences only (no paged cache at all), a loop over everything that starts at layer 0.
CFG_C = {"architecture": "Lofudra", "vocab": 64, "width": 32, "norm": {"eps": 1e-6},
         "loop": {"start": 0, "stop": 2, "times": 3},
         "layers": [layer(mlstm(4, 8, 8, 15.0), 48), layer(mamba2(2, 16, 24, 2, 5, 2), None)]}
# D: attention without a window over a head size of 128 (long prompts take the tiled kernel, long contexts split their
# keys, and the sink enters where the splits are merged), one key head, no rotation; a loop of one pass.
CFG_D = {"architecture": "Lofudra", "vocab": 150, "width": 64, "norm": {"eps": 1e-6},
         "loop": {"start": 1, "stop": 2, "times": 1},
         "layers": [layer(parallel(left(2, 1, 128, 0.09, turned=0), right(2, 32, 8, [0.5, 0.97]), 0.9, 0.9), 40),
                    layer(parallel(left(1, 1, 32, 0.2, window=1, base=100.0), right(3, 8, 8, [1.0, 0.0, 0.8]), 1.5, 0.4), 40)]}
# E: sizes that fit no vector width: a width of 50, a head size of 12 (the plain attention kernels in both precisions),
# five query heads, state sizes of 20 and 10, seven taps, a window of 17.
CFG_E = {"architecture": "Lofudra", "vocab": 101, "width": 50, "norm": {"eps": 1e-5},
         "loop": {"start": 1, "stop": 2, "times": 2},
         "layers": [layer(parallel(left(5, 5, 12, 0.4, window=17, base=777.0, turned=6), right(3, 10, 14, [0.98, 0.6, 0.9999]), 0.5, 2.0), 30),
                    layer(mamba2(5, 6, 20, 1, 7, 5), 30),
                    layer(mlstm(3, 10, 14, 8.0), 30)]}
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C, "D": CFG_D, "E": CFG_E}


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    """Every tensor of a model, from the design."""
    W, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    loop = cfg.get("loop")
    if loop:
        out["loop.step"] = (loop["times"], W)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        out[p + "norm1"] = out[p + "norm1b"] = (W,)
        if L["type"] == "parallel":
            a, r = m["left"], m["right"]
            out.update({p + "mix.left.q": (a["heads"] * a["dim"], W), p + "mix.left.q.b": (a["heads"] * a["dim"],),
                        p + "mix.left.k": (a["kv_heads"] * a["dim"], W), p + "mix.left.k.b": (a["kv_heads"] * a["dim"],),
                        p + "mix.left.q.norm": (a["dim"],), p + "mix.left.k.norm": (a["dim"],),
                        p + "mix.left.o": (W, a["heads"] * a["vdim"]),
                        p + "mix.right.q": (r["heads"] * r["dim"], W), p + "mix.right.k": (r["heads"] * r["dim"], W),
                        p + "mix.right.v": (r["heads"] * r["vdim"], W), p + "mix.right.g": (r["heads"] * r["vdim"], W),
                        p + "mix.right.o": (W, r["heads"] * r["vdim"])})
        elif L["type"] == "mlstm":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * d, W), p + "mix.k": (H * d, W), p + "mix.v": (H * dv, W), p + "mix.g": (H * dv, W),
                        p + "mix.o": (W, H * dv), p + "mix.norm": (H * dv,), p + "mix.i": (H, W), p + "mix.i.b": (H,),
                        p + "mix.f": (H, W), p + "mix.f.b": (H,)})
        else:
            H, dv, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = H * dv, H * dv + 2 * G * N
            out.update({p + "mix.in": (2 * inner + 2 * G * N + H, W), p + "mix.conv": (ch, m["conv"]), p + "mix.conv.b": (ch,),
                        p + "mix.dt_bias": (H,), p + "mix.A_log": (H,), p + "mix.D": (H,), p + "mix.norm": (inner,),
                        p + "mix.o": (W, inner)})
        if L["mlp"] is not None:
            out[p + "norm2"] = out[p + "norm2b"] = (W,)
            out[p + "mlp.up"], out[p + "mlp.down"] = (L["mlp"]["ff"], W), (W, L["mlp"]["ff"])
    return out


def random_weights(cfg: dict, seed: int, sharpen: float = 1.0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and name[1].isdigit() else name
        if leaf in ("norm1", "norm2", "mix.norm", "mix.left.q.norm", "mix.left.k.norm") or name == "final.norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf in ("norm1b", "norm2b"):
            t = 0.5 + 0.1 * torch.randn(shape, generator=g)                 # (what a sub-layer adds to the stream)
        elif leaf == "mix.A_log":
            t = torch.empty(shape).uniform_(-6.0, 1.0, generator=g)         # rates from remembering for hundreds of tokens to forgetting
        elif leaf == "mix.dt_bias":
            t = torch.empty(shape).uniform_(-3.0, 1.0, generator=g)
        elif leaf == "mix.D":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf == "mix.f.b":
            t = torch.empty(shape).uniform_(1.0, 6.0, generator=g)          # forget gates near 1: a long memory
        elif leaf.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif leaf == "mix.conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif name == "loop.step":
            t = 0.5 * torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
            if leaf == "mix.left.q":
                t = t * sharpen
            if leaf in ("mix.i", "mix.f"):
                t = t * 3.0                                                  # so that the gates' caps bite now and then
        out[name] = t.to(dtype)
    return out


def write_model(folder: str, cfg: dict, seed: int, sharpen: float = 1.0) -> Dict[str, torch.Tensor]:
    from inferrs_amd.weights import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    weights = random_weights(cfg, seed, sharpen)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights)
    return weights


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
