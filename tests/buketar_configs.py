"""Tiny Buketar configurations that differ in every size and option, and random weights for them.

The tensor list is written out here from the design (not asked of the package), so a part that expects
another name or shape fails to load.  Weights are drawn so that the mechanisms matter: matrices N(0, 1/in),
stream connections near (but not at) the identity, decays spread from forgetting at once to remembering for
hundreds of tokens; `sharpen` multiplies the query projections so that a query singles out a few keys somewhere
in its context, and a key that is lost or read from a wrong page changes the logits by far more than rounding."""
from __future__ import annotations

import json
import os
from typing import Dict

import torch


def attention(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, turned=None, scaling=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": rot_dim if turned is None else turned, "scaling": scaling}}}


def recurrence(width, blocks, conv):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}}


def moe(ff, experts, top, scale, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "scale": scale}}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}

# A: two streams, a looped pair, part of the rotated features turning under the YaRN law, value size other than
# the key's, a cached row of 48 (a size the matrix-core attention takes in bfloat16).
CFG_A = {"architecture": "Buketar", "vocab": 211, "width": 48, "norm": {"eps": 1e-5}, "streams": 2, "logit_softcap": 12.0,
         "loop": {"start": 1, "stop": 3, "times": 2},
         "layers": [layer(recurrence(40, 2, 4), moe(24, 5, 2, 1.5, 2.0)),
                    layer(attention(3, 24, 8, 20, 40, 0.2, base=5000.0, turned=4, scaling=YARN), moe(24, 5, 2, 1.5, 2.0)),
                    layer(recurrence(40, 2, 4), None),
                    layer(attention(3, 24, 8, 20, 40, 0.2, base=5000.0, turned=4, scaling=YARN), moe(16, 3, 3, 0.7, 0.5))]}
# B: no stream connections, no loop, no cap; a cached row of 34 (the plain attention kernels in both precisions), a
# single head, no scaling law, one block, two taps, a router that takes one expert of many.
CFG_B = {"architecture": "Buketar", "vocab": 97, "width": 40, "norm": {"eps": 1e-6},
         "layers": [layer(attention(1, 16, 6, 12, 28, 0.3), moe(20, 9, 1, 2.5, 1.0)),
                    layer(recurrence(56, 1, 2), moe(20, 9, 1, 2.5, 1.0)),
                    layer(attention(1, 16, 6, 12, 28, 0.3), None)]}
# C: recurrences only (no paged cache at all), a single stream with connections, one tap, a loop over everything.
CFG_C = {"architecture": "Buketar", "vocab": 64, "width": 32, "norm": {"eps": 1e-6}, "streams": 1, "logit_softcap": 30.0,
         "loop": {"start": 0, "stop": 2, "times": 3},
         "layers": [layer(recurrence(48, 3, 1), moe(16, 4, 4, 1.0, 3.0)), layer(recurrence(32, 4, 5), None)]}
# D: attention only, four streams, many heads on a wide cached row (128: matrix cores in bfloat16), a loop of one pass.
CFG_D = {"architecture": "Buketar", "vocab": 150, "width": 64, "norm": {"eps": 1e-6}, "streams": 4,
         "loop": {"start": 0, "stop": 1, "times": 1},
         "layers": [layer(attention(8, 16, 32, 24, 96, 0.15, base=100.0, scaling={"factor": 16.0, "original": 32, "fast": 4.0, "slow": 2.0}),
                          moe(40, 6, 3, 2.0, 1.0)),
                    layer(attention(2, 40, 16, 8, 16, 0.1, base=1e6, turned=16), moe(40, 6, 3, 2.0, 1.0))]}
# E: sizes that fit no vector width: a model width of 50, experts of 30, a recurrence of 42 channels in blocks of 14, a
# cached row of 28, five heads, three streams, seven experts of which a token runs five.
CFG_E = {"architecture": "Buketar", "vocab": 101, "width": 50, "norm": {"eps": 1e-5}, "streams": 3, "logit_softcap": 20.0,
         "loop": {"start": 1, "stop": 2, "times": 2},
         "layers": [layer(attention(5, 12, 6, 10, 22, 0.25, base=777.0, turned=2), moe(30, 7, 5, 1.2, 1.5)),
                    layer(recurrence(42, 3, 3), moe(30, 7, 5, 1.2, 1.5))]}
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C, "D": CFG_D, "E": CFG_E}


def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    """Every tensor of a model, from the design."""
    W, V, S = cfg["width"], cfg["vocab"], cfg.get("streams")
    out = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        subs = [1] if L["mlp"] is None else [1, 2]
        for q in subs:
            out[f"{p}norm{q}"] = (W,)
            out[f"{p}ls{q}"] = (W,)
            if S:
                out[f"{p}hc{q}.in"], out[f"{p}hc{q}.out"], out[f"{p}hc{q}.mix"] = (S,), (S,), (S, S)
        if L["type"] == "latent_attention":
            H, d, r, dv, k = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            out.update({p + "mix.q": (H * (d + r), W), p + "mix.dkv": (k + r, W), p + "mix.dkv.norm": (k,),
                        p + "mix.uk": (H * d, k), p + "mix.uv": (H * dv, k), p + "mix.g": (H * dv, W), p + "mix.o": (W, H * dv)})
        else:
            w, b = m["width"], m["blocks"]
            out.update({p + "mix.y": (w, W), p + "mix.y.b": (w,), p + "mix.x": (w, W), p + "mix.x.b": (w,),
                        p + "mix.conv": (w, m["conv"]), p + "mix.conv.b": (w,), p + "mix.ra": (b, w // b, w // b),
                        p + "mix.ra.b": (b, w // b), p + "mix.ri": (b, w // b, w // b), p + "mix.ri.b": (b, w // b),
                        p + "mix.lam": (w,), p + "mix.o": (W, w)})
        if L["mlp"] is not None:
            ff, E = L["mlp"]["expert"]["ff"], L["mlp"]["router"]["experts"]
            out[p + "mlp.router"] = (E, W)
            for e in range(E):
                out.update({f"{p}mlp.e{e}.gate": (ff, W), f"{p}mlp.e{e}.up": (ff, W), f"{p}mlp.e{e}.down": (W, ff)})
    return out


def random_weights(cfg: dict, seed: int, sharpen: float = 1.0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        if leaf in ("norm1", "norm2", "ls1", "ls2", "mix.dkv.norm") or name == "final.norm":
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif leaf.endswith(".mix") and "hc" in leaf:
            t = torch.eye(shape[0]) * 0.8 + 0.25 * torch.randn(shape, generator=g)
        elif leaf.endswith(".in") or leaf.endswith(".out"):
            t = 0.8 + 0.3 * torch.randn(shape, generator=g)
        elif leaf == "mix.lam":
            t = torch.empty(shape).uniform_(-7.0, 1.0, generator=g)        # decays from a = 0.99.. down to forgetting
        elif leaf.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif leaf == "mix.conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif leaf == "mlp.router":
            t = 2.0 * torch.randn(shape, generator=g) / shape[-1] ** 0.5
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
            if leaf == "mix.q":
                t = t * sharpen
            if leaf.endswith(".gate") or leaf.endswith(".up"):
                t = t * 1.5                                                 # so that the experts' clamps bite now and then
        out[name] = t.to(dtype)
    return out


def write_model(folder: str, cfg: dict, seed: int, sharpen: float = 1.0) -> str:
    from inferrs_amd.weights import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), random_weights(cfg, seed, sharpen))
    return folder


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
