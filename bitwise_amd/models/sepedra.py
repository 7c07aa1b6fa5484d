"""The Sepedra decoder as a ModelSpec: layers x += norm1(mixer(x)); x += norm2(ff(x)) (the norm behind the sublayer,
the sublayers read the stream itself) whose mixers are, layer by layer, gated attention with a convolution behind its
projections (some layers read another layer's cache) or a real-gated linear recurrent unit; feed-forwards of routed
experts; a final norm and an untied head whose logits are soft-capped.  Layer i's tensors start with ``l<i>.``: norm1,
norm2, mix.*, mlp.*; the rest are ``embed``, ``final.norm`` and ``head``."""

from __future__ import annotations

from ..config.sepedra import SepedraConfig
from ..parts.base import LayerCall, LayerSpec, ModelSpec, PartSpec

# A small configuration for simulations and smoke runs: sizes that are all different, a layer that reads another's
# cache, a layer without feed-forward, fewer key heads than query heads, a partly rotated head, values narrower than keys.
TINY_SEPEDRA = {
    "architecture": "Sepedra", "vocab": 97, "width": 40, "norm": {"eps": 1e-5}, "logit_softcap": 20.0, "max_positions": 512,
    "eos_token_id": 2,
    "layers": [
        {"type": "rglru", "mixer": {"width": 24, "blocks": 3, "conv": 4},
         "mlp": {"kind": "moe", "expert": {"ff": 16, "limit": 2.0}, "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}}},
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "conv": 3, "scale": 0.4,
                   "rot": {"base": 1000.0, "dims": 8, "scaling": {"factor": 2.0, "low": 1.0, "high": 4.0, "original": 64}}},
         "mlp": None},
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "conv": 2, "scale": 0.3, "kv_from": 1,
                   "rot": {"base": 1000.0, "dims": 8, "scaling": {"factor": 2.0, "low": 1.0, "high": 4.0, "original": 64}}},
         "mlp": {"kind": "moe", "expert": {"ff": 24, "limit": 1.5}, "router": {"experts": 4, "top": 3}}},
    ],
}


def sepedra_spec(cfg: SepedraConfig) -> ModelSpec:
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        pre = f"l{i}."
        m = dict(layer.mixer)
        cache = i
        if layer.type == "attention":
            rot = dict(m["rot"])
            shared = m.get("kv_from") is not None
            if shared:
                cache = int(m["kv_from"])
            params = {"width": cfg.width, "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]),
                      "vdim": int(m["vdim"]), "scale": float(m["scale"]), "eps": cfg.eps, "conv": int(m["conv"]),
                      "qk_norm": True, "sink": 0.0, "gate": True, "shared_kv": shared, "window": None,
                      "position": PartSpec("rope_pairs", {"base": float(rot["base"]), "dims": int(rot["dims"]),
                                                          "scaling": rot.get("scaling"), "max_positions": cfg.max_positions})}
            mixer = PartSpec("gated_attention", params, pre + "mix.")
            schedule.append(LayerCall(layer=i, cache=cache, writes_cache=not shared))
        else:
            mixer = PartSpec("rglru", {"width": cfg.width, "inner": int(m["width"]), "blocks": int(m["blocks"]),
                                       "conv": int(m["conv"]), "decay_scale": 8.0}, pre + "mix.")
            schedule.append(LayerCall(layer=i, cache=i))
        parts = {
            "mixer_norm": PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps, "tensor": "norm1"}, pre),
            "mixer": mixer,
        }
        if layer.mlp is not None:
            ex, ro = layer.mlp["expert"], layer.mlp["router"]
            groups = ro.get("groups") or {"count": 1, "keep": 1}
            parts["ffn_norm"] = PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps, "tensor": "norm2"}, pre)
            parts["feed_forward"] = PartSpec("moe", {"width": cfg.width, "experts": int(ro["experts"]), "top": int(ro["top"]),
                                                     "groups": int(groups["count"]), "keep": int(groups["keep"]),
                                                     "ff": int(ex["ff"]), "limit": float(ex["limit"]), "alpha": 1.702}, pre + "mlp.")
        layers.append(LayerSpec("postnorm", parts))
    return ModelSpec(
        architecture=cfg.architecture,
        vocab_size=cfg.vocab,
        width=cfg.width,
        embedding=PartSpec("embedding", {"vocab": cfg.vocab, "width": cfg.width, "tensor": "embed"}, ""),
        layers=layers,
        schedule=schedule,
        final_norm=PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps, "tensor": "norm"}, "final."),
        lm_head=PartSpec("lm_head_softcap", {"vocab": cfg.vocab, "width": cfg.width, "tied": False, "tensor": "head",
                                             "cap": cfg.logit_softcap}, ""),
        max_positions=cfg.max_positions,
        bos_token_id=cfg.bos_token_id,
        eos_token_id=cfg.eos_token_id,
    )
