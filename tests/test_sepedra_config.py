"""The Sepedra configuration and registry on the CPU: keys read from config.json, refusals, the tensors a configuration
names, the schedule of layers that read another layer's cache, and the stretched rotary frequencies."""

import copy

import numpy as np
import pytest

import plain_sepedra as ps
from bitwise_amd.config.llama import ConfigError
from bitwise_amd.config.sepedra import SepedraConfig
from bitwise_amd.model import describe, model_spec
from bitwise_amd.models.sepedra import TINY_SEPEDRA
from bitwise_amd.registry import ARCHITECTURES, architecture_of


def test_registry_and_round_trip():
    arch = architecture_of(TINY_SEPEDRA)
    assert arch is ARCHITECTURES["Sepedra"] and arch.tiny_config is TINY_SEPEDRA
    cfg = SepedraConfig.from_dict(TINY_SEPEDRA)
    again = SepedraConfig.from_dict(cfg.to_dict())
    assert again == cfg and cfg.layers[2].mixer["kv_from"] == 1 and cfg.layers[1].mlp is None
    assert cfg.logit_softcap == 20.0 and cfg.eps == 1e-5


def test_tensor_names_and_schedule():
    spec = model_spec(TINY_SEPEDRA)
    t = describe(TINY_SEPEDRA)
    assert t["embed"].shape == (97, 40) and t["head"].shape == (97, 40) and t["final.norm"].shape == (40,)
    assert t["l0.mix.ra"].shape == (3, 8, 8) and t["l0.mix.conv"].shape == (24, 4) and t["l0.mix.lam"].shape == (24,)
    assert t["l0.mlp.router"].shape == (6, 40) and t["l0.mlp.e5.down"].shape == (40, 16) and "l0.mlp.e6.gate" not in t
    assert t["l1.mix.k"].shape == (32, 40) and t["l1.mix.v"].shape == (16, 40) and t["l1.mix.v.conv"].shape == (16, 3)
    assert t["l1.mix.g"].shape == (32, 40) and t["l1.mix.o"].shape == (40, 32) and "l1.norm2" not in t
    # a layer that reads another's cache has queries, their convolution, the gate and the output projection only
    assert "l2.mix.k" not in t and "l2.mix.v.conv" not in t and t["l2.mix.q.conv"].shape == (64, 2)
    calls = spec.schedule
    assert [(c.layer, c.cache, c.writes_cache) for c in calls] == [(0, 0, True), (1, 1, True), (2, 1, False)]
    assert spec.lm_head.kind == "lm_head_softcap" and spec.lm_head.params["cap"] == 20.0
    assert all(l.block == "postnorm" for l in spec.layers)


@pytest.mark.parametrize("change, what", [
    (lambda c: c.pop("logit_softcap"), "logit_softcap"),
    (lambda c: c["layers"][0].update(type="mamba"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][1]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=0), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=16), "kv_from"),
    (lambda c: c["layers"][0]["mixer"].update(blocks=5), "blocks"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "experts"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
])
def test_refusals(change, what):
    cfg = copy.deepcopy(TINY_SEPEDRA)
    change(cfg)
    with pytest.raises(ConfigError) as e:
        SepedraConfig.from_dict(cfg)
    assert what in str(e.value)


def test_stretched_frequencies_on_the_host():
    from bitwise_amd.parts.rope import PairRotaryTable
    from bitwise_amd.runtime import Runtime
    for rot in ({"base": 2000.0, "dims": 20, "scaling": {"factor": 5.0, "low": 1.0, "high": 8.0, "original": 96}},
                {"base": 10000.0, "dims": 6}, {"base": 50.0, "dims": 2, "scaling": {"factor": 2.0, "low": 2.0, "high": 3.0, "original": 10}}):
        table = PairRotaryTable({"base": rot["base"], "dims": rot["dims"], "scaling": rot.get("scaling"), "max_positions": 4},
                                Runtime("float32", device=None))
        assert np.allclose(table.frequencies(), ps.rotary_frequencies(rot).numpy(), rtol=1e-14)
