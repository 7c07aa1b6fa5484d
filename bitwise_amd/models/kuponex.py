"""The Kuponex decoder as a ModelSpec: parallel layers x += mixer(shift(norm1(x))) + ff(norm2(x)) whose mixers are,
layer by layer, a matrix LSTM, gated linear attention or attention over a compressed cache; norms whose weights
are kept as their distance from 1; a gated GELU feed-forward; a final norm and an untied head.  Layer i's tensors start with
``l<i>.``: norm1, norm2, shift, mix.*, mlp.{gate,up,down}; the rest are ``embed``, ``final.norm`` and ``head``."""

from __future__ import annotations

from ..config.kuponex import KuponexConfig
from ..parts.base import LayerCall, LayerSpec, ModelSpec, PartSpec

# A small configuration for simulations and smoke runs: one layer of each mixer, sizes that are all different.
TINY_KUPONEX = {
    "architecture": "Kuponex", "vocab": 89, "width": 48, "norm": {"eps": 1e-5}, "max_positions": 512, "eos_token_id": 2,
    "layers": [
        {"type": "gla", "mixer": {"heads": 2, "dim": 8, "vdim": 24, "tau": 8.0, "rank": 4}, "mlp": {"kind": "dense", "ff": 96}},
        {"type": "latent_attention",
         "mixer": {"heads": 3, "dim": 8, "rot_dim": 4, "vdim": 12, "kv_rank": 20, "scale": 0.25, "rot": {"base": 1000.0, "dims": 4}},
         "mlp": {"kind": "dense", "ff": 64}},
        {"type": "mlstm", "mixer": {"heads": 2, "dim": 12, "vdim": 16, "gate_cap": 10.0}, "mlp": None},
    ],
}


def kuponex_spec(cfg: KuponexConfig) -> ModelSpec:
    layers = []
    for i, layer in enumerate(cfg.layers):
        pre = f"l{i}."
        m = dict(layer.mixer)
        params = {"width": cfg.width, "eps": cfg.eps, "heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m["vdim"])}
        if layer.type == "mlstm":
            params["gate_cap"] = float(m["gate_cap"])
        elif layer.type == "gla":
            params.update(tau=float(m["tau"]), rank=int(m["rank"]))
        else:
            params.update(rot_dim=int(m["rot_dim"]), kv_rank=int(m["kv_rank"]), scale=float(m["scale"]), window=m.get("window"),
                          position=PartSpec("rope", {"theta": float(m["rot"]["base"]), "head_dim": int(m["rot"]["dims"]),
                                                     "max_positions": cfg.max_positions}))
        parts = {
            "mixer_norm": PartSpec("rmsnorm_shift", {"width": cfg.width, "eps": cfg.eps, "offset": 1.0, "tensor": "norm1",
                                                      "mix_tensor": "shift"}, pre),
            "mixer": PartSpec(layer.type, params, pre + "mix."),
        }
        if layer.ff is not None:
            parts["ffn_norm"] = PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps, "offset": 1.0, "tensor": "norm2"}, pre)
            parts["feed_forward"] = PartSpec("geglu", {"width": cfg.width, "inter": layer.ff}, pre + "mlp.")
        layers.append(LayerSpec("parallel", parts))
    return ModelSpec(
        architecture=cfg.architecture,
        vocab_size=cfg.vocab,
        width=cfg.width,
        embedding=PartSpec("embedding", {"vocab": cfg.vocab, "width": cfg.width, "tensor": "embed"}, ""),
        layers=layers,
        schedule=[LayerCall(layer=i, cache=i) for i in range(len(layers))],
        final_norm=PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps, "offset": 1.0, "tensor": "norm"}, "final."),
        lm_head=PartSpec("lm_head", {"vocab": cfg.vocab, "width": cfg.width, "tied": False, "tensor": "head"}, ""),
        max_positions=cfg.max_positions,
        bos_token_id=cfg.bos_token_id,
        eos_token_id=cfg.eos_token_id,
    )
