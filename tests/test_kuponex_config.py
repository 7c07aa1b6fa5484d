"""Kuponex without a GPU: its configuration reader, registry entry, tensor names, and the plain implementation's
own consistency (its recurrences against their unrolled sums)."""

import json

import pytest
import torch

import plain_kuponex as pk
from bitwise_amd import registry
from bitwise_amd.config.kuponex import KuponexConfig, sizes_from_tensors
from bitwise_amd.config.llama import ConfigError
from bitwise_amd.model import describe, write_random_model

CFG = {
    "architecture": "Kuponex", "vocab": 53, "width": 32, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "gla", "mixer": {"heads": 2, "dim": 4, "vdim": 6, "tau": 4.0}, "mlp": {"kind": "dense", "ff": 40}},
        {"type": "latent_attention", "mlp": None,
         "mixer": {"heads": 2, "dim": 4, "rot_dim": 4, "vdim": 6, "kv_rank": 10, "scale": 0.3, "rot": {"base": 100.0, "dims": 4}}},
        {"type": "mlstm", "mixer": {"heads": 1, "dim": 4, "vdim": 8, "gate_cap": 5.0}, "mlp": {"kind": "dense", "ff": 24}},
    ],
}


def with_rank(cfg, rank):
    return sizes_from_tensors(cfg, {"l0.mix.a1": (rank, cfg["width"])})


def test_registry_reads_the_architecture_by_its_single_name():
    arch = registry.architecture_of(CFG)
    assert arch.name == "Kuponex" and arch.tiny_config is not None
    typed = arch.config_from_dict(with_rank(CFG, 3))
    assert isinstance(typed, KuponexConfig) and typed.layers[0].mixer["rank"] == 3 and typed.layers[1].ff is None
    assert KuponexConfig.from_dict(typed.to_dict()) == typed
    with pytest.raises(ConfigError, match="rank"):
        arch.config_from_dict(CFG)                       # no checkpoint to take the inner size from
    bad = json.loads(json.dumps(CFG))
    bad["layers"][2]["type"] = "conv"
    with pytest.raises(ConfigError, match="type"):
        arch.config_from_dict(with_rank(bad, 3))
    bad = json.loads(json.dumps(CFG))
    del bad["layers"][1]["mixer"]["kv_rank"]
    with pytest.raises(ConfigError, match="kv_rank"):
        arch.config_from_dict(with_rank(bad, 3))


def test_tensor_names_and_a_folder_that_completes_its_own_sizes(tmp_path):
    cfg = with_rank(CFG, 5)
    names = describe(cfg)
    assert names["embed"].shape == (53, 32) and names["final.norm"].shape == (32,) and names["head"].shape == (53, 32)
    assert names["l0.mix.a1"].shape == (5, 32) and names["l0.mix.a2"].shape == (8, 5) and names["l0.mix.norm"].shape == (6,)
    assert names["l1.mix.dkv"].shape == (14, 32) and names["l1.mix.uv"].shape == (12, 10) and names["l1.mix.sink"].shape == (2,)
    assert names["l2.mix.norm"].shape == (8,) and names["l2.mix.f.b"].shape == (1,) and names["l0.shift"].shape == (32,)
    assert "l1.mlp.gate" not in names and "l1.norm2" not in names and names["l2.mlp.down"].shape == (32, 24)
    folder = write_random_model(tmp_path / "m", cfg, 3, 0.1)
    stored = json.loads((folder / "config.json").read_text())
    del stored["layers"][0]["mixer"]["rank"]            # as a checkpoint that only its tensors tell the size
    (folder / "config.json").write_text(json.dumps(stored))
    assert registry.read_model_config(folder)["layers"][0]["mixer"]["rank"] == 5


def test_plain_recurrences_equal_their_unrolled_sums():
    """gla: S_t = sum_s (prod_{s<r<=t} alpha_r) k_s v_s^T; token shift and the norm on the side."""
    g = torch.Generator().manual_seed(1)
    cfg = with_rank(CFG, 3)
    from bitwise_amd.weights.loader import random_tensors
    w = pk.to64(dict(random_tensors(describe(cfg), 4, 0.3, torch.float32)))
    T = 9
    h = torch.randn(T, 32, generator=g, dtype=torch.float64)
    m = cfg["layers"][0]["mixer"]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["l0.mix.q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w["l0.mix.k"].T).view(T, H, D)
    v = (h @ w["l0.mix.v"].T).view(T, H, V)
    alpha = torch.sigmoid((h @ w["l0.mix.a1"].T) @ w["l0.mix.a2"].T + w["l0.mix.a2.b"]).pow(1 / m["tau"]).view(T, H, D)
    o = torch.zeros(T, H, V, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            decay = alpha[s + 1:t + 1].prod(0)
            o[t] += torch.einsum("hd,hd,hv->hv", q[t] * decay, k[s], v[s])
    o = pk.rms_unit(o, 1e-5) * w["l0.mix.norm"]
    want = (o.reshape(T, H * V) * torch.nn.functional.silu(h @ w["l0.mix.g"].T)) @ w["l0.mix.o"].T
    assert torch.allclose(pk.gla_mixer(h, w, "l0.", m, 1e-5), want, rtol=1e-10, atol=1e-12)
    shifted = pk.token_shift(h, torch.full((32,), 0.25, dtype=torch.float64))
    assert torch.allclose(shifted[0], 0.75 * h[0]) and torch.allclose(shifted[3], 0.75 * h[3] + 0.25 * h[2])
    x = torch.randn(2, 32, generator=g, dtype=torch.float64)
    assert torch.allclose(pk.norm_around_zero(x, torch.zeros(32, dtype=torch.float64), 0.0).pow(2).mean(-1), torch.ones(2, dtype=torch.float64))
    lg = pk.forward(cfg, w, [1, 2, 3, 4, 5])
    assert lg.shape == (5, 53) and torch.allclose(pk.forward(cfg, w, [1, 2, 3])[-1], lg[2])     # causal
