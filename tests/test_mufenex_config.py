"""Mufenex on the CPU: its config.json typed and written back, the spec it becomes, the tensors
it declares, and the plain implementation's formulas pinned by values worked out by hand."""
import copy
import math

import pytest
import torch

import plain_mufenex as plain
from mufenex_models import MODELS
from xinfer_amd.config.model_config import ConfigError
from xinfer_amd.engine.model import CausalLM
from xinfer_amd.models import config_from_dict
from xinfer_amd.models.mufenex import head_slopes


@pytest.mark.parametrize("name", list(MODELS))
def test_config_round_trip_and_spec(name):
    raw = MODELS[name]["config"]
    fam, cfg = config_from_dict(raw)
    assert fam.name == "mufenex"
    assert fam.config_class.from_dict(cfg.to_dict()) == cfg
    spec = fam.spec(cfg)
    assert len(spec.layers) == len(raw["layers"]) and spec.vocab_size == raw["vocab"]
    mixing = [i for i, l in enumerate(raw["layers"]) if l["mixer"].get("v_mix")]
    for i, (l, r) in enumerate(zip(spec.layers, raw["layers"])):
        m = r["mixer"]
        assert l.block == "branchnorm" and l.mixer.kind == "attention"
        assert l.mixer["value_dim"] == m["vdim"] and l.mixer["head_dim"] == m["dim"]
        assert l.mixer["window"] == (m.get("mask") or {}).get("size")
        assert l.mixer["score_softcap"] == m.get("softcap")
        assert len(l.mixer["distance_slopes"]) == m["heads"]
        vm = l.mixer.get("value_mix")
        assert (vm is not None) == bool(m.get("v_mix"))
        if vm:
            assert vm["source"] == (i == mixing[0])
        assert (l.feed_forward is None) == (r["mlp"] is None)
        if r["mlp"]:
            assert l.feed_forward.kind == ("gated_mlp" if r["mlp"]["kind"] == "dense" else "routed_experts")
    names = {d.name: tuple(d.shape) for d in CausalLM.declare(spec)}
    assert names["embed"] == (raw["vocab"], raw["width"]) and names["head"] == (raw["vocab"], raw["width"])
    for i, r in enumerate(raw["layers"]):
        m = r["mixer"]
        assert names[f"l{i}.mix.q"] == (m["heads"] * m["dim"], raw["width"])
        assert names[f"l{i}.mix.v"] == (m["kv_heads"] * m["vdim"], raw["width"])
        assert names[f"l{i}.mix.o"] == (raw["width"], m["heads"] * m["vdim"])
        assert names[f"l{i}.mix.q.norm"] == (m["heads"] * m["dim"],)
        assert names[f"l{i}.mix.k.norm"] == (m["kv_heads"] * m["dim"],)
        assert (f"l{i}.mix.vmix" in names) == (bool(m.get("v_mix")) and i != mixing[0])
        assert (f"l{i}.norm2" in names) == (r["mlp"] is not None)
        if r["mlp"] and r["mlp"]["kind"] == "moe":
            e = r["mlp"]["router"]["experts"]
            assert names[f"l{i}.mlp.router"] == (e, raw["width"]) and names[f"l{i}.mlp.router.b"] == (e,)
            assert names[f"l{i}.mlp.e{e - 1}.down"] == (raw["width"], r["mlp"]["expert"]["ff"])
            assert f"l{i}.mlp.e{e}.down" not in names


def test_config_errors():
    base = MODELS["P"]["config"]
    for change, text in [
        (lambda c: c["layers"][0].__setitem__("type", "recurrent"), "unknown layer type"),
        (lambda c: c["layers"][1]["mlp"].__setitem__("kind", "sparse"), "unknown mlp kind"),
        (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 9), "experts cannot be chosen"),
        (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 4), "cannot be run"),
        (lambda c: c["layers"][2]["mixer"].__setitem__("vdim", 16), "different sizes"),
        (lambda c: c.pop("vocab"), "vocab"),
        (lambda c: c["norm"].pop("eps"), "eps"),
    ]:
        raw = copy.deepcopy(base)
        change(raw)
        with pytest.raises(ConfigError, match=text):
            config_from_dict(raw)


def test_slopes():
    assert head_slopes(4) == (0.25, 0.0625, 0.015625, 0.00390625)
    assert head_slopes(1) == (2.0 ** -8,)
    for h in range(6):
        assert plain.head_slope(h, 6) == pytest.approx(head_slopes(6)[h])


def test_plain_formulas():
    # sinusoid: row p, entries (sin, cos) of p * 10000^(-2i / width)
    pe = plain.sinusoid_positions(3, 4, torch.float64)
    assert pe[0].tolist() == [0.0, 1.0, 0.0, 1.0]
    assert pe[2, 0].item() == pytest.approx(math.sin(2.0)) and pe[2, 1].item() == pytest.approx(math.cos(2.0))
    assert pe[2, 2].item() == pytest.approx(math.sin(2.0 / 100.0)) and pe[2, 3].item() == pytest.approx(math.cos(0.02))
    # norm: eps inside the root
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert plain.rms_norm(x, 0.5)[0].tolist() == pytest.approx([3.0 / math.sqrt(13.0), 4.0 / math.sqrt(13.0)])
    # gelu, tanh form
    assert plain.gelu_tanh(torch.tensor(1.0, dtype=torch.float64)).item() == pytest.approx(0.8411919906082768)
    # window: the query sees itself and the window - 1 keys before it
    v = plain.visible(1, 10, 9, 4)
    assert v[0].tolist() == [False] * 6 + [True] * 4
    # scores: cap, then the distance bias, then the softmax over the visible keys
    q = torch.tensor([[2.0]], dtype=torch.float64)
    k = torch.tensor([[1.0], [3.0], [5.0]], dtype=torch.float64)
    p = plain.scores(q, k, 0.5, 2.0, 0.25, 2, first_q=2)
    s1, s2 = 2.0 * math.tanh(3.0 / 2.0) - 0.25, 2.0 * math.tanh(5.0 / 2.0)
    assert p[0, 0].item() == 0.0
    assert p[0, 1].item() == pytest.approx(math.exp(s1) / (math.exp(s1) + math.exp(s2)))
    # the router's weights are the softmax over the chosen logits only
    W = {"r.router": torch.tensor([[1.0], [3.0], [2.0]], dtype=torch.float64), "r.router.b": torch.tensor([0.0, 0.0, 1.5], dtype=torch.float64)}
    idx, wt = plain.route(torch.tensor([[1.0]], dtype=torch.float64), W, "r.", 2)
    assert idx[0].tolist() == [2, 1] and wt[0, 0].item() == pytest.approx(1.0 / (1.0 + math.exp(-0.5)))
    # blended values
    assert plain.blend_values(torch.tensor(2.0), torch.tensor(10.0), torch.tensor(0.25)).item() == pytest.approx(4.0)


def test_random_model_folder_loads_in_the_plain_implementation(tmp_path):
    from mufenex_models import make_model, router_margin, MARGIN
    d = make_model(str(tmp_path / "Q"), "Q")
    pm = plain.PlainMufenex(d)
    toks = list(range(1, 61))
    lg = pm.logits(toks)
    assert lg.shape == (60, 257) and torch.isfinite(lg).all()
    assert router_margin(d, toks) >= 0.8 * MARGIN
    # tokens that no chain of windows reaches change nothing: the layers see 8 + 8 + 16 + 8 positions back
    other = [200] * 10 + toks[10:]
    assert torch.allclose(pm.logits(other)[-1], lg[-1], atol=1e-5)
    assert not torch.allclose(pm.logits([200] * 25 + toks[25:])[-1], lg[-1], atol=1e-5)
