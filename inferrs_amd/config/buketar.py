"""Configuration of the Buketar decoder, read from its config.json.

config.json describes the model layer by layer:

    "architecture": "Buketar", "vocab", "width", "norm": {"eps"}, "logit_softcap" (optional),
    "streams" (optional: the number of residual streams with learned connections between them),
    "loop": {"start", "stop", "times"} (optional: layers start..stop-1 run `times` times in a row, each
    pass with a cache or state of its own),
    "layers": [{"type": "latent_attention" | "rglru", "mixer": {...}, "mlp": {...} | null}, ...]

    mixer of "latent_attention": heads, dim, rot_dim, vdim, kv_rank, scale,
                                 rot: {base, dims, scaling: {factor, original, fast, slow} | null}
    mixer of "rglru":            width, blocks, conv
    mlp: {"kind": "moe", "expert": {ff, limit}, "router": {experts, top, scale}}

Every size and every constant that differs from model to model comes from there; what the design fixes
(the recurrence's decay constant 8, the experts' activation constant 1.702, the sigmoid router without
renormalisation) stands in `to_spec`.  Tensor names: "embed", "head", "final.norm", and for layer i
"l<i>.norm1|norm2", "l<i>.ls1|ls2", "l<i>.hc1|hc2.in|out|mix", "l<i>.mix.*", "l<i>.mlp.*".
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, Tuple

from .base import ConfigError
from .spec import (CappedHeadSpec, GatedRecurrenceSpec, LatentAttentionSpec, LayerSpec, ModelSpec, NormSpec,
                   PositionSpec, RoutedExpertsSpec, ScheduleEntry, StreamsSpec)

DEFAULT_MAX_POSITION = 1 << 17
RECURRENCE_DECAY = 8.0
EXPERT_ALPHA = 1.702


def _get(d: Dict[str, Any], key: str, where: str, kind=(int, float), minimum=None):
    if not isinstance(d, dict) or key not in d or d[key] is None:
        raise ConfigError(f"config.json: required key '{where}.{key}' is missing")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError(f"config.json: '{where}.{key}' has the wrong type: {v!r}")
    if minimum is not None and v < minimum:
        raise ConfigError(f"config.json: '{where}.{key}' must be >= {minimum}, got {v}")
    return v


def _int(d, key, where, minimum=1) -> int:
    return int(_get(d, key, where, (int,), minimum))


def _num(d, key, where) -> float:
    return float(_get(d, key, where))


@dataclass(frozen=True)
class BuketarConfig:
    raw: Any                        # config.json as read (a dictionary), checked by `from_dict`

    architecture = "Buketar"
    model_type = "buketar"
    chat_template = None

    # ---- reading ----------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict[str, Any], allow_ignored_keys: bool = False) -> "BuketarConfig":
        cfg = cls(copy.deepcopy(raw))
        cfg.to_spec()                # every key is read and checked there
        return cfg

    def to_dict(self) -> Dict[str, Any]:
        out = copy.deepcopy(self.raw)
        out.setdefault("architecture", self.architecture)
        return out

    @property
    def vocab_size(self) -> int:
        return _int(self.raw, "vocab", "")

    @property
    def hidden_size(self) -> int:
        return _int(self.raw, "width", "")

    @property
    def eos_token_ids(self) -> Tuple[int, ...]:
        return ()

    def run_order(self) -> Tuple[int, ...]:
        """The layers in the order they run (a looped range several times in a row)."""
        n = len(self.raw.get("layers") or [])
        loop = self.raw.get("loop")
        if not loop:
            return tuple(range(n))
        start, stop, times = _int(loop, "start", "loop", 0), _int(loop, "stop", "loop", 0), _int(loop, "times", "loop", 1)
        if not (0 <= start <= stop <= n):
            raise ConfigError(f"config.json: 'loop' {start}..{stop} lies outside the {n} layers")
        return tuple(range(start)) + tuple(range(start, stop)) * times + tuple(range(stop, n))

    # ---- the model as data --------------------------------------------------------------------
    def _mixer(self, i: int, layer: Dict[str, Any], hidden: int, eps: float):
        where = f"layers[{i}].mixer"
        kind, m = layer.get("type"), layer.get("mixer")
        if kind == "latent_attention":
            rot_dim = _int(m, "rot_dim", where, 0)
            rot = m.get("rot") or {}
            turned = _int(rot, "dims", where + ".rot", 0) if rot_dim else 0
            if turned > rot_dim or turned % 2:
                raise ConfigError(f"config.json: '{where}.rot.dims' = {turned} must be even and within rot_dim {rot_dim}")
            scaling = None
            sc = rot.get("scaling") if rot_dim else None
            if sc:
                w = where + ".rot.scaling"
                scaling = ("yarn", _num(sc, "factor", w), _num(sc, "original", w), _num(sc, "fast", w), _num(sc, "slow", w))
            position = (PositionSpec("rope", head_dim=rot_dim, rot_dim=turned, theta=_num(rot, "base", where + ".rot"),
                                     pairing="half", scaling=scaling) if turned else PositionSpec("none"))
            return LatentAttentionSpec(hidden=hidden, n_heads=_int(m, "heads", where), head_dim=_int(m, "dim", where),
                                       rot_dim=rot_dim, v_dim=_int(m, "vdim", where), kv_rank=_int(m, "kv_rank", where),
                                       position=position, scale=_num(m, "scale", where), norm_eps=eps, gate=True)
        if kind == "rglru":
            width, blocks = _int(m, "width", where), _int(m, "blocks", where)
            if width % blocks:
                raise ConfigError(f"config.json: '{where}.width' = {width} is no multiple of its {blocks} blocks")
            return GatedRecurrenceSpec(hidden=hidden, width=width, blocks=blocks, conv=_int(m, "conv", where),
                                       decay=RECURRENCE_DECAY)
        raise ConfigError(f"config.json: layers[{i}].type = {kind!r} is no mixer of this design "
                          "(known: 'latent_attention', 'rglru')")

    def _mlp(self, i: int, layer: Dict[str, Any], hidden: int):
        f = layer.get("mlp")
        if f is None:
            return None
        where = f"layers[{i}].mlp"
        if f.get("kind") != "moe":
            raise ConfigError(f"config.json: '{where}.kind' = {f.get('kind')!r} is no feed-forward of this design (known: 'moe')")
        expert, router = f.get("expert"), f.get("router")
        experts, top = _int(router, "experts", where + ".router"), _int(router, "top", where + ".router")
        if top > experts:
            raise ConfigError(f"config.json: '{where}.router.top' = {top} exceeds its {experts} experts")
        return RoutedExpertsSpec(hidden=hidden, intermediate=_int(expert, "ff", where + ".expert"), experts=experts, top=top,
                                 scale=_num(router, "scale", where + ".router"), limit=_num(expert, "limit", where + ".expert"),
                                 alpha=EXPERT_ALPHA, score="sigmoid", renormalize=False)

    def to_spec(self) -> ModelSpec:
        raw = self.raw
        if not isinstance(raw, dict):
            raise ConfigError("config.json must hold an object")
        vocab, hidden = self.vocab_size, self.hidden_size
        eps = _num(raw.get("norm"), "eps", "norm")
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        streams = raw.get("streams")
        if streams is not None:
            streams = _int(raw, "streams", "")
        norm = NormSpec(hidden, eps)
        layers = []
        for i, layer in enumerate(layers_raw):
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
            p = f"l{i}."
            ffn = self._mlp(i, layer, hidden)
            n_norms = 1 if ffn is None else 2
            layers.append(LayerSpec(
                mixer=self._mixer(i, layer, hidden, eps), ffn=ffn, norms=(norm,) * n_norms,
                norm_names=tuple(f"{p}norm{q + 1}" for q in range(n_norms)), mixer_prefix=p + "mix.", ffn_prefix=p + "mlp.",
                arrangement="streams",
                residual=StreamsSpec(streams=streams or 1, hidden=hidden, prefix=p, connections=streams is not None,
                                     layer_scale=True)))
        cap = raw.get("logit_softcap")
        if cap is not None:
            cap = _num(raw, "logit_softcap", "")
            if cap <= 0:
                raise ConfigError(f"config.json: 'logit_softcap' must be positive, got {cap}")
        max_position = int(raw.get("max_position") or DEFAULT_MAX_POSITION)
        return ModelSpec(
            architecture=self.architecture, vocab_size=vocab, hidden=hidden, layers=tuple(layers),
            schedule=tuple(ScheduleEntry(i) for i in self.run_order()),
            final_norm=norm, final_norm_name="final.norm", embed_name="embed", head_name="head",
            max_position=max_position, head_required=True, eos_token_ids=(),
            head=CappedHeadSpec(vocab, hidden, "head", cap))
