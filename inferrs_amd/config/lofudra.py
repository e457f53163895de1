"""Configuration of the Lofudra decoder, read from its config.json.

config.json describes the model layer by layer:

    "architecture": "Lofudra", "vocab", "width", "norm": {"eps"},
    "loop": {"start", "stop", "times"} (optional: the layers from `start` up to but not including `stop` are walked
    `times` times over before the model goes on, every walk keeping caches and states of its own; row t of the tensor
    "loop.step" enters the stream ahead of walk t, and ahead of every walk but the first so does the embedding's output),
    "layers": [{"type": "parallel" | "mlstm" | "mamba2", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | null}, ...]

    mixer of "parallel": left: {heads, kv_heads, dim, vdim, scale, mask: {size}, rot: {base, dims}},
                         right: {heads, dim, vdim, decay: [one a head]}, left_scale, right_scale
    mixer of "mlstm":    heads, dim, vdim, gate_cap
    mixer of "mamba2":   heads, vdim, state, groups, conv, norm_groups

Every size and every constant that differs from model to model comes from there; what the design fixes (the sink in the
left softmax, values that are the keys, the exact GELU, norms on both sides of every sub-layer) stands in `to_spec`.
Tensor names: "embed", "head", "final.norm", "loop.step", and for layer i "l<i>.norm1|norm1b|norm2|norm2b",
"l<i>.mix.*", "l<i>.mlp.up|down".
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, Tuple

from .base import ConfigError
from .buketar import _int, _num
from .spec import (AttentionSpec, DenseMlpSpec, LayerSpec, MatrixMemorySpec, ModelSpec, NormSpec, PassInputSpec,
                   PositionSpec, RetentionSpec, ScheduleEntry, SideBySideSpec, StateSpaceSpec)

DEFAULT_MAX_POSITION = 1 << 17

# the left mixer's tensors as the attention part names them -> as the file names them
LEFT_NAMES = (("q_proj.weight", "q"), ("q_proj.bias", "q.b"), ("k_proj.weight", "k"), ("k_proj.bias", "k.b"),
              ("q_norm.weight", "q.norm"), ("k_norm.weight", "k.norm"), ("o_proj.weight", "o"))


@dataclass(frozen=True)
class LofudraConfig:
    raw: Any                        # config.json as read (a dictionary), checked by `from_dict`

    architecture = "Lofudra"
    model_type = "lofudra"
    chat_template = None

    # ---- reading ----------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict[str, Any], allow_ignored_keys: bool = False) -> "LofudraConfig":
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

    def schedule(self) -> Tuple[ScheduleEntry, ...]:
        """The layers in the order they run; the first stop of every pass over the looped range is marked."""
        n = len(self.raw.get("layers") or [])
        loop = self.raw.get("loop")
        if not loop:
            return tuple(ScheduleEntry(i) for i in range(n))
        start, stop, times = _int(loop, "start", "loop", 0), _int(loop, "stop", "loop", 0), _int(loop, "times", "loop", 1)
        if not (0 <= start <= stop <= n):
            raise ConfigError(f"config.json: 'loop' {start}..{stop} lies outside the {n} layers")
        out = [ScheduleEntry(i) for i in range(start)]
        for t in range(times):
            out += [ScheduleEntry(i, pass_index=t if i == start else None) for i in range(start, stop)]
        return tuple(out + [ScheduleEntry(i) for i in range(stop, n)])

    def loop_times(self) -> int:
        """Passes over the looped range (0: no loop, or an empty range)."""
        loop = self.raw.get("loop")
        if not loop or _int(loop, "start", "loop", 0) >= _int(loop, "stop", "loop", 0):
            return 0
        return _int(loop, "times", "loop", 1)

    # ---- the model as data --------------------------------------------------------------------
    def _left(self, m: Dict[str, Any], where: str, hidden: int, eps: float) -> AttentionSpec:
        dim = _int(m, "dim", where)
        vdim = _int(m, "vdim", where) if m.get("vdim") is not None else dim
        if vdim != dim:
            raise ConfigError(f"config.json: '{where}.vdim' = {vdim} differs from 'dim' = {dim}, but the values are the keys")
        heads, kv_heads = _int(m, "heads", where), _int(m, "kv_heads", where)
        if heads % kv_heads:
            raise ConfigError(f"config.json: '{where}.heads' = {heads} is no multiple of 'kv_heads' = {kv_heads}")
        rot = m.get("rot") or {}
        turned = _int(rot, "dims", where + ".rot", 0) if rot else 0
        if turned > dim or turned % 2:
            raise ConfigError(f"config.json: '{where}.rot.dims' = {turned} must be even and within dim {dim}")
        position = (PositionSpec("rope", head_dim=dim, rot_dim=turned, theta=_num(rot, "base", where + ".rot"), pairing="half")
                    if turned else PositionSpec("none"))
        mask = m.get("mask") or {}
        window = _int(mask, "size", where + ".mask") if mask else None
        return AttentionSpec(hidden=hidden, n_heads=heads, n_kv_heads=kv_heads, head_dim=dim, position=position,
                             qk_norm=NormSpec(dim, eps), window=window, scale=_num(m, "scale", where), qkv_bias=True,
                             sink=True, values_from_keys=True, names=LEFT_NAMES)

    def _right(self, m: Dict[str, Any], where: str, hidden: int, eps: float) -> RetentionSpec:
        heads = _int(m, "heads", where)
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError(f"config.json: '{where}.decay' must list one number for each of the {heads} heads")
        return RetentionSpec(hidden=hidden, n_heads=heads, head_dim=_int(m, "dim", where), v_dim=_int(m, "vdim", where),
                             decay=tuple(float(d) for d in decay), norm_eps=eps)

    def _mixer(self, i: int, layer: Dict[str, Any], hidden: int, eps: float):
        where = f"layers[{i}].mixer"
        kind, m = layer.get("type"), layer.get("mixer")
        if not isinstance(m, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        if kind == "parallel":
            for side in ("left", "right"):
                if not isinstance(m.get(side), dict):
                    raise ConfigError(f"config.json: required key '{where}.{side}' is missing")
            return SideBySideSpec(left=self._left(m["left"], where + ".left", hidden, eps),
                                  right=self._right(m["right"], where + ".right", hidden, eps),
                                  left_scale=_num(m, "left_scale", where), right_scale=_num(m, "right_scale", where))
        if kind == "mlstm":
            return MatrixMemorySpec(hidden=hidden, n_heads=_int(m, "heads", where), head_dim=_int(m, "dim", where),
                                    v_dim=_int(m, "vdim", where), gate_cap=_num(m, "gate_cap", where), norm_eps=eps)
        if kind == "mamba2":
            heads, groups, vdim = _int(m, "heads", where), _int(m, "groups", where), _int(m, "vdim", where)
            norm_groups = _int(m, "norm_groups", where)
            if heads % groups:
                raise ConfigError(f"config.json: '{where}.heads' = {heads} is no multiple of 'groups' = {groups}")
            if (heads * vdim) % norm_groups:
                raise ConfigError(f"config.json: '{where}.norm_groups' = {norm_groups} does not divide heads * vdim = {heads * vdim}")
            return StateSpaceSpec(hidden=hidden, n_heads=heads, v_dim=vdim, state=_int(m, "state", where), groups=groups,
                                  conv=_int(m, "conv", where), norm_groups=norm_groups, norm_eps=eps)
        raise ConfigError(f"config.json: layers[{i}].type = {kind!r} is no mixer of this design "
                          "(known: 'parallel', 'mlstm', 'mamba2')")

    def _mlp(self, i: int, layer: Dict[str, Any], hidden: int):
        f = layer.get("mlp")
        if f is None:
            return None
        where = f"layers[{i}].mlp"
        if not isinstance(f, dict) or f.get("kind") != "dense":
            raise ConfigError(f"config.json: '{where}.kind' is no feed-forward of this design (known: 'dense')")
        return DenseMlpSpec(hidden=hidden, intermediate=_int(f, "ff", where), activation="gelu")

    def to_spec(self) -> ModelSpec:
        raw = self.raw
        if not isinstance(raw, dict):
            raise ConfigError("config.json must hold an object")
        vocab, hidden = self.vocab_size, self.hidden_size
        eps = _num(raw.get("norm"), "eps", "norm")
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        norm = NormSpec(hidden, eps)
        layers = []
        for i, layer in enumerate(layers_raw):
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
            p = f"l{i}."
            ffn = self._mlp(i, layer, hidden)
            names = (p + "norm1", p + "norm1b") + ((p + "norm2", p + "norm2b") if ffn is not None else ())
            layers.append(LayerSpec(mixer=self._mixer(i, layer, hidden, eps), ffn=ffn, norms=(norm,) * len(names),
                                    norm_names=names, mixer_prefix=p + "mix.", ffn_prefix=p + "mlp.",
                                    arrangement="sandwich_norm"))
        times = self.loop_times()
        max_position = int(raw.get("max_position") or DEFAULT_MAX_POSITION)
        return ModelSpec(
            architecture=self.architecture, vocab_size=vocab, hidden=hidden, layers=tuple(layers), schedule=self.schedule(),
            final_norm=norm, final_norm_name="final.norm", embed_name="embed", head_name="head",
            max_position=max_position, head_required=True, eos_token_ids=(),
            pass_input=PassInputSpec("loop.step", times, hidden, readd_embedding=True) if times else None)
