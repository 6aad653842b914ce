"""Lilalorn's configuration and its turning into a model description, on the CPU."""
import copy

import pytest
import torch

from lilalorn_models import MODELS, make_model
from xinfer_amd.config.model_config import ConfigError
from xinfer_amd.models import config_from_dict, family_of, load_config


def test_config_round_trip_and_registry():
    for name, t in MODELS.items():
        fam, cfg = config_from_dict(t["config"])
        assert fam is family_of("Lilalorn") and cfg.architecture == "Lilalorn"
        assert fam.config_class.from_dict(cfg.to_dict()) == cfg
        assert len(cfg.layers) == len(t["config"]["layers"])


def test_spec_has_a_run_for_every_layer_and_tensors_once():
    from xinfer_amd.engine.model import CausalLM
    fam, cfg = config_from_dict(MODELS["A"]["config"])
    spec = fam.spec(cfg)
    assert [(e.layer, e.cache_id) for e in spec.schedule] == [(0, None), (1, None), (0, 3), (2, None), (1, 4)]
    assert [l.prefix for l in spec.layers] == ["l0", "l1", "l3"]
    assert spec.layers[2].feed_forward is None and list(spec.layers[2].norms) == ["norm1"]
    assert all(l.block == "prenorm" and l.block_params["residual_scale"] == 0.6 for l in spec.layers)
    assert spec.head["scale"] == 0.4
    names = [d.name for d in CausalLM.declare(spec)]
    assert len(names) == len(set(names))
    for want in ("embed", "l0.mix.left.q", "l0.mix.right.g", "l0.mlp.e4.up", "l0.mlp.shared.sg", "l1.mix.a2.b", "l1.mix.norm",
                 "l3.mix.right.o", "final.norm", "head"):
        assert want in names
    assert not any(n.startswith(("l2.", "l4.", "l3.mlp", "l3.norm2")) for n in names)
    model = CausalLM(spec, torch.float32)
    # every run has a state of its own, the parallel ones pages too; all keys are kept: one group
    assert sorted(model.state_needs) == [0, 1, 2, 3, 4] and sorted(model.kv_needs) == [0, 2, 3]
    assert [g.window for g in model.cache_groups] == [0]
    assert model.state_needs[3].shape == (3, 8, 16) and model.state_needs[4].shape == (2, 16, 24)
    left = spec.layers[0].mixer["branches"][0][2]
    assert left["position"]["scaling"] == dict(kind="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original=64.0)
    assert left["position"]["rotary_dim"] == 8 and left["value_dim"] == 24


def test_the_decay_rank_is_the_checkpoints(tmp_path):
    from xinfer_amd.engine.loading import ShapedNames
    from xinfer_amd.weights.store import SafetensorsStore
    d = make_model(str(tmp_path / "O"), "O")
    fam, cfg = load_config(d)
    store = SafetensorsStore(d)
    try:
        spec = fam.spec(cfg, ShapedNames(store))
    finally:
        store.close()
    assert spec.layers[1].mixer["decay_rank"] == 5 and fam.spec(cfg).layers[1].mixer["decay_rank"] == 32


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="conv"), "unknown layer type"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5]), "decays"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=4), "kv heads"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=64), "rotated dims"),
    (lambda c: c["layers"][1]["mixer"].update(tau=0.0), "tau"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "experts"),
    (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
    (lambda c: c["layers"][2].update(weights_of=11), "weights_of"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_configurations_that_cannot_be_run(change, message):
    raw = copy.deepcopy(MODELS["A"]["config"])
    change(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw)
