"""Typed configuration of the Kuponex decoder, read from the keys of its config.json.

Keys: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps``, and ``layers``: a list whose entries give
``type`` (the mixer: "mlstm", "gla" or "latent_attention"), ``mixer`` (its sizes and constants) and ``mlp``
({"kind": "dense", "ff": n} or null for a layer without feed-forward).  Mixer keys:

* mlstm: heads, dim, vdim, gate_cap
* gla: heads, dim, vdim, tau; ``rank`` (the inner size of the decay's low-rank projection) may be given, and is
  otherwise the number of rows of the layer's ``mix.a1`` tensor
* latent_attention: heads, dim, rot_dim, vdim, kv_rank, scale, rot = {base, dims}; optional window

Optional keys with defaults that a checkpoint's config.json need not carry: ``max_positions`` (the length of the
rotary tables and the longest request), ``bos_token_id``, ``eos_token_id``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .llama import ConfigError

ARCHITECTURE = "Kuponex"
MIXER_KEYS = {
    "mlstm": ("heads", "dim", "vdim", "gate_cap"),
    "gla": ("heads", "dim", "vdim", "tau"),
    "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"),
}
DEFAULT_MAX_POSITIONS = 1 << 16


def _positive_int(d: Mapping[str, Any], key: str, where: str) -> int:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or v < 1:
        raise ConfigError(f"config.json: {where} needs a positive integer '{key}', got {v!r}")
    return v


@dataclass(frozen=True)
class KuponexLayer:
    type: str
    mixer: Mapping[str, Any]
    ff: Optional[int]                 # None: the layer has no feed-forward


@dataclass(frozen=True)
class KuponexConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    layers: Tuple[KuponexLayer, ...]
    max_positions: int
    bos_token_id: int
    eos_token_id: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "KuponexConfig":
        name = d.get("architecture")
        if not isinstance(name, str):
            raise ConfigError("config.json lacks 'architecture': name")
        norm = d.get("norm")
        if not isinstance(norm, Mapping) or "eps" not in norm:
            raise ConfigError("config.json lacks 'norm': {'eps': ...}")
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json lacks a non-empty list 'layers'")
        layers: List[KuponexLayer] = []
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
            for k in ("heads", "dim", "vdim"):
                _positive_int(mixer, k, where)
            if kind == "gla":
                if "rank" not in mixer:
                    raise ConfigError(f"config.json: {where} (gla) gives no 'rank' and no checkpoint was there to take it from")
                _positive_int(mixer, "rank", where)
            if kind == "latent_attention":
                for k in ("rot_dim", "kv_rank"):
                    _positive_int(mixer, k, where)
                rot = mixer["rot"]
                if not isinstance(rot, Mapping) or "base" not in rot or "dims" not in rot:
                    raise ConfigError(f"config.json: {where} needs rot = {{base, dims}}")
                if int(rot["dims"]) % 2 or not 0 < int(rot["dims"]) <= int(mixer["rot_dim"]):
                    raise ConfigError(f"config.json: {where}: rot.dims must be even and at most rot_dim")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where} has an mlp of kind {mlp.get('kind') if isinstance(mlp, Mapping) else mlp!r}; known: dense")
                ff = _positive_int(mlp, "ff", where + " mlp")
            layers.append(KuponexLayer(kind, copy.deepcopy(dict(mixer)), ff))
        eos, bos = d.get("eos_token_id", -1), d.get("bos_token_id", -1)
        return cls(architecture=name, vocab=_positive_int(d, "vocab", "the model"), width=_positive_int(d, "width", "the model"),
                   eps=float(norm["eps"]), layers=tuple(layers),
                   max_positions=int(d.get("max_positions", DEFAULT_MAX_POSITIONS)),
                   bos_token_id=-1 if bos is None else int(bos), eos_token_id=-1 if eos is None else int(eos))

    def to_dict(self) -> Dict[str, Any]:
        return {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
            "layers": [{"type": l.type, "mixer": copy.deepcopy(dict(l.mixer)),
                        "mlp": None if l.ff is None else {"kind": "dense", "ff": l.ff}} for l in self.layers],
            "max_positions": self.max_positions, "bos_token_id": self.bos_token_id, "eos_token_id": self.eos_token_id,
        }


def sizes_from_tensors(config: Mapping[str, Any], shapes: Mapping[str, Tuple[int, ...]]) -> Dict[str, Any]:
    """The configuration with the sizes that only the checkpoint's tensor shapes give filled in: a gla layer's ``rank``."""
    out = copy.deepcopy(dict(config))
    for i, entry in enumerate(out.get("layers") or []):
        if isinstance(entry, dict) and entry.get("type") == "gla" and isinstance(entry.get("mixer"), dict):
            shape = shapes.get(f"l{i}.mix.a1")
            if "rank" not in entry["mixer"] and shape is not None and len(shape) == 2:
                entry["mixer"]["rank"] = int(shape[0])
    return out
