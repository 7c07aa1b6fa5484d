"""Typed configuration of the Sepedra decoder, read from the keys of its config.json.

Keys: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps``, ``logit_softcap``, and ``layers``: a list whose
entries give ``type`` (the mixer: "attention" or "rglru"), ``mixer`` (its sizes and constants) and ``mlp`` (the
feed-forward, or null for a layer without one).  Mixer keys:

* attention: heads, kv_heads, dim, vdim, conv (taps of the convolution behind the projections), scale,
  rot = {base, dims, scaling = {factor, low, high, original} or absent}; optional kv_from (the layer whose cached keys
  and values this layer reads instead of making its own)
* rglru: width (the channels of its two branches), blocks, conv

mlp: {"kind": "moe", "expert": {ff, limit}, "router": {experts, top, groups = {count, keep} or absent}}.

Optional keys with defaults that a checkpoint's config.json need not carry: ``max_positions`` (the length of the
rotary tables and the longest request), ``bos_token_id``, ``eos_token_id``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .llama import ConfigError

ARCHITECTURE = "Sepedra"
MIXER_KEYS = {
    "attention": ("heads", "kv_heads", "dim", "vdim", "conv", "scale", "rot"),
    "rglru": ("width", "blocks", "conv"),
}
DEFAULT_MAX_POSITIONS = 1 << 16


def _positive_int(d: Mapping[str, Any], key: str, where: str) -> int:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or v < 1:
        raise ConfigError(f"config.json: {where} needs a positive integer '{key}', got {v!r}")
    return v


@dataclass(frozen=True)
class SepedraLayer:
    type: str
    mixer: Mapping[str, Any]
    mlp: Optional[Mapping[str, Any]]          # None: the layer has no feed-forward


@dataclass(frozen=True)
class SepedraConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    logit_softcap: float
    layers: Tuple[SepedraLayer, ...]
    max_positions: int
    bos_token_id: int
    eos_token_id: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "SepedraConfig":
        name = d.get("architecture")
        if not isinstance(name, str):
            raise ConfigError("config.json lacks 'architecture': name")
        norm = d.get("norm")
        if not isinstance(norm, Mapping) or "eps" not in norm:
            raise ConfigError("config.json lacks 'norm': {'eps': ...}")
        if "logit_softcap" not in d or not float(d["logit_softcap"]) > 0:
            raise ConfigError("config.json lacks a positive 'logit_softcap'")
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json lacks a non-empty list 'layers'")
        layers: List[SepedraLayer] = []
        for i, entry in enumerate(raw_layers):
            where = f"layer {i}"
            kind = entry.get("type") if isinstance(entry, Mapping) else None
            if kind not in MIXER_KEYS:
                raise ConfigError(f"config.json: {where} has type {kind!r}; known: {sorted(MIXER_KEYS)}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, Mapping):
                raise ConfigError(f"config.json: {where} lacks 'mixer'")
            missing = [k for k in MIXER_KEYS[kind] if k not in mixer]
            if missing:
                raise ConfigError(f"config.json: {where} ({kind}) lacks mixer keys {missing}")
            _positive_int(mixer, "conv", where)
            if kind == "attention":
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    _positive_int(mixer, k, where)
                if int(mixer["heads"]) % int(mixer["kv_heads"]):
                    raise ConfigError(f"config.json: {where}: heads must be a multiple of kv_heads")
                rot = mixer["rot"]
                if not isinstance(rot, Mapping) or "base" not in rot or "dims" not in rot:
                    raise ConfigError(f"config.json: {where} needs rot = {{base, dims}}")
                if int(rot["dims"]) % 2 or not 0 <= int(rot["dims"]) <= int(mixer["dim"]):
                    raise ConfigError(f"config.json: {where}: rot.dims must be even and at most dim")
                sc = rot.get("scaling")
                if sc is not None and (not isinstance(sc, Mapping) or any(k not in sc for k in ("factor", "low", "high", "original"))):
                    raise ConfigError(f"config.json: {where}: rot.scaling needs factor, low, high and original")
                src = mixer.get("kv_from")
                if src is not None:
                    ok = isinstance(src, int) and not isinstance(src, bool) and 0 <= src < i and layers[src].type == "attention" \
                        and layers[src].mixer.get("kv_from") is None
                    if not ok:
                        raise ConfigError(f"config.json: {where}: kv_from must name an earlier attention layer with keys and values of its own")
                    other = layers[src].mixer
                    if any(other[k] != mixer[k] for k in ("kv_heads", "dim", "vdim")) or dict(other["rot"]) != dict(rot):
                        raise ConfigError(f"config.json: {where}: kv_from names a layer with other key/value heads or another rotation")
            else:
                for k in ("width", "blocks"):
                    _positive_int(mixer, k, where)
                if int(mixer["width"]) % int(mixer["blocks"]):
                    raise ConfigError(f"config.json: {where}: width must be a multiple of blocks")
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") != "moe":
                    raise ConfigError(f"config.json: {where} has an mlp of kind {mlp.get('kind') if isinstance(mlp, Mapping) else mlp!r}; known: moe")
                ex, ro = mlp.get("expert"), mlp.get("router")
                if not isinstance(ex, Mapping) or not isinstance(ro, Mapping) or "limit" not in ex:
                    raise ConfigError(f"config.json: {where} mlp needs expert = {{ff, limit}} and router = {{experts, top}}")
                _positive_int(ex, "ff", where + " mlp.expert")
                experts, top = _positive_int(ro, "experts", where + " mlp.router"), _positive_int(ro, "top", where + " mlp.router")
                groups = ro.get("groups")
                count, keep = 1, 1
                if groups is not None:
                    count, keep = _positive_int(groups, "count", where + " mlp.router.groups"), _positive_int(groups, "keep", where + " mlp.router.groups")
                if experts % count or keep > count or top > keep * (experts // count):
                    raise ConfigError(f"config.json: {where}: {top} of {experts} experts in {count} groups of which {keep} are kept does not work out")
            layers.append(SepedraLayer(kind, copy.deepcopy(dict(mixer)), None if mlp is None else copy.deepcopy(dict(mlp))))
        eos, bos = d.get("eos_token_id", -1), d.get("bos_token_id", -1)
        return cls(architecture=name, vocab=_positive_int(d, "vocab", "the model"), width=_positive_int(d, "width", "the model"),
                   eps=float(norm["eps"]), logit_softcap=float(d["logit_softcap"]), layers=tuple(layers),
                   max_positions=int(d.get("max_positions", DEFAULT_MAX_POSITIONS)),
                   bos_token_id=-1 if bos is None else int(bos), eos_token_id=-1 if eos is None else int(eos))

    def to_dict(self) -> Dict[str, Any]:
        return {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
            "logit_softcap": self.logit_softcap,
            "layers": [{"type": l.type, "mixer": copy.deepcopy(dict(l.mixer)),
                        "mlp": None if l.mlp is None else copy.deepcopy(dict(l.mlp))} for l in self.layers],
            "max_positions": self.max_positions, "bos_token_id": self.bos_token_id, "eos_token_id": self.eos_token_id,
        }
