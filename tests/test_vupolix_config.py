"""The Vupolix configuration and registry on the CPU: keys read from config.json, refusals, the tensors a configuration
names, the order in which looped layers run, the plain implementation's own mechanisms on small cases worked by hand,
and a model folder written and read back (with the one size that only a tensor's shape gives)."""

import copy
import json
import math

import pytest
import torch

import plain_vupolix as pv
from bitwise_amd.config.llama import ConfigError
from bitwise_amd.config.vupolix import VupolixConfig
from bitwise_amd.model import describe, model_spec, write_random_model
from bitwise_amd.models.vupolix import TINY_VUPOLIX
from bitwise_amd.registry import ARCHITECTURES, architecture_of, read_model_config


def test_registry_and_round_trip():
    arch = architecture_of(TINY_VUPOLIX)
    assert arch is ARCHITECTURES["Vupolix"] and arch.tiny_config is TINY_VUPOLIX
    cfg = VupolixConfig.from_dict(TINY_VUPOLIX)
    again = VupolixConfig.from_dict(cfg.to_dict())
    assert again == cfg and cfg.layers[1].mlp is None and cfg.loop == (1, 3, 3)
    assert cfg.logit_scale == 0.7 and cfg.residual_mult == 0.4
    bare = copy.deepcopy(TINY_VUPOLIX)
    bare.pop("loop")
    assert VupolixConfig.from_dict(bare).loop == (0, 0, 1)


def test_order_of_layer_runs():
    cfg = VupolixConfig.from_dict(TINY_VUPOLIX)
    runs = cfg.layer_runs()
    assert runs == [(0, False), (1, False), (2, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    assert runs == pv.layer_runs(TINY_VUPOLIX)
    spec = model_spec(TINY_VUPOLIX)
    assert [(c.layer, c.adds_embedding) for c in spec.schedule] == runs
    assert [c.cache for c in spec.schedule] == list(range(8))          # every run has a cache and state of its own
    once = copy.deepcopy(TINY_VUPOLIX)
    once["loop"] = {"start": 2, "stop": 2, "times": 5}
    assert [c.layer for c in model_spec(once).schedule] == [0, 1, 2, 3]
    whole = copy.deepcopy(TINY_VUPOLIX)
    whole["loop"] = {"start": 0, "stop": 4, "times": 2}
    assert [(c.layer, c.adds_embedding) for c in model_spec(whole).schedule] == [(0, False), (1, False), (2, False), (3, False),
                                                                                 (0, True), (1, False), (2, False), (3, False)]


def test_tensor_names_and_parts():
    spec = model_spec(TINY_VUPOLIX)
    t = describe(TINY_VUPOLIX)
    assert t["embed"].shape == (89, 40) and t["embed.norm"].shape == (40,) and t["head"].shape == (89, 40)
    assert t["final.norm"].shape == (40,)
    for n in ("norm1", "norm1b", "norm2", "norm2b"):
        assert t["l0." + n].shape == (40,)
    assert "l1.norm2" not in t and "l1.norm2b" not in t and "l1.norm1b" in t
    assert t["l0.mix.left.q"].shape == (64, 40) and t["l0.mix.left.k"].shape == (32, 40) and "l0.mix.left.v" not in t
    assert t["l0.mix.left.sink"].shape == (4,) and t["l0.mix.left.g"].shape == (4, 40) and t["l0.mix.left.o"].shape == (40, 64)
    assert t["l0.mix.right.q"].shape == (16, 40) and t["l0.mix.right.v"].shape == (48, 40) and t["l0.mix.right.g"].shape == (48, 40)
    assert t["l0.mix.right.o"].shape == (40, 48) and "l0.mix.right.norm" not in t
    assert t["l0.mix.left.out"].shape == (40,) and t["l0.mix.right.out"].shape == (40,)
    for s in "rkvgw":
        assert t["l1.mix.mu." + s].shape == (40,)
    assert t["l1.mix.r"].shape == (24, 40) and t["l1.mix.w1"].shape == (5, 40) and t["l1.mix.w2"].shape == (24, 5)
    assert t["l1.mix.w0"].shape == (24,) and t["l1.mix.u"].shape == (3, 8) and t["l1.mix.norm"].shape == (24,) and t["l1.mix.o"].shape == (40, 24)
    assert t["l0.mlp.router"].shape == (6, 40) and t["l0.mlp.correction"].shape == (6,) and t["l0.mlp.e5.down"].shape == (40, 16)
    assert t["l0.mlp.shared.up"].shape == (24, 40) and "l0.mlp.shared.sg" not in t and "l2.mlp.shared.gate" not in t
    assert all(l.block == "sandwich" for l in spec.layers)
    assert spec.layers[0].parts["mixer_post_norm"].params["scale"] == 0.4 and spec.layers[0].parts["ffn_post_norm"].params["scale"] == 0.4
    assert spec.layers[1].parts["mixer_norm"].kind == "rmsnorm_shift" and spec.layers[0].parts["mixer_norm"].kind == "rmsnorm"
    left = dict(spec.layers[0].mixer.params["branches"])["left"].params
    assert left["window"] == 24 and left["sink"] == "learned" and left["gate"] == "head" and left["values"] == "keys"
    ff = spec.layers[0].parts["feed_forward"].params
    assert ff["score"] == "sigmoid" and ff["correction"] and ff["group_best"] == 2 and (ff["groups"], ff["keep"]) == (3, 2)
    assert spec.lm_head.params["scale"] == 0.7 and not spec.lm_head.params["tied"]


@pytest.mark.parametrize("change, what", [
    (lambda c: c.pop("residual_mult"), "residual_mult"),
    (lambda c: c.pop("logit_scale"), "logit_scale"),
    (lambda c: c["loop"].update(stop=5), "loop"),
    (lambda c: c["loop"].update(times=0), "loop"),
    (lambda c: c["layers"][0].update(type="mamba"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("dim"), "dim"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(vdim=8), "vdim"),
    (lambda c: c["layers"][0]["mixer"]["left"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"]["scaling"].pop("fast"), "scaling"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.9]), "decay"),
    (lambda c: c["layers"][2]["mlp"]["router"].update(top=5), "experts"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
])
def test_refusals(change, what):
    cfg = copy.deepcopy(TINY_VUPOLIX)
    change(cfg)
    with pytest.raises(ConfigError) as e:
        VupolixConfig.from_dict(cfg)
    assert what in str(e.value)


def test_a_model_folder_comes_back(tmp_path):
    from bitwise_amd.weights import loader
    folder = write_random_model(tmp_path / "m", TINY_VUPOLIX, 5, 0.1)
    # a checkpoint's config.json need not say the decay projection's inner size: the tensor's rows do
    raw = json.loads((folder / "config.json").read_text())
    for layer in raw["layers"]:
        layer["mixer"].pop("rank", None)
    (folder / "config.json").write_text(json.dumps(raw))
    raw = read_model_config(folder)
    assert VupolixConfig.from_dict(raw) == VupolixConfig.from_dict(TINY_VUPOLIX)
    w = loader.load_folder(folder, describe(raw))
    assert w["l1.mix.w1"].shape == (5, 40) and w["l3.mix.w1"].shape == (3, 40) and w["l0.mlp.correction"].shape == (6,)


def test_the_plain_mechanisms_by_hand():
    F = pv.F
    # the shift: the first token mixes with zeros
    h = torch.tensor([[2.0], [4.0]], dtype=F)
    assert pv.shifted(h, torch.tensor([0.25], dtype=F)).tolist() == [[1.5], [3.5]]
    # the memory with a bonus: the first token reads nothing but its own k v through the bonus
    r, k, v = (torch.tensor([[[x]], [[y]]], dtype=F) for x, y in ((1.0, 2.0), (3.0, 5.0), (7.0, 11.0)))
    decay, bonus = torch.full((2, 1, 1), 0.5, dtype=F), torch.tensor([[0.1]], dtype=F)
    out = pv.wkv_recurrence(r, k, v, decay, bonus)
    assert abs(float(out[0]) - 0.1 * 3 * 7 * 1) < 1e-12 and abs(float(out[1]) - (3 * 7 + 0.1 * 5 * 11) * 2) < 1e-12
    # retention reads after the update
    out = pv.retention(r, k, v, [0.5])
    assert float(out[0]) == 21.0 and float(out[1]) == (0.5 * 21 + 55) * 2
    # a window of 2 and a sink of zero: one key of score 0 and the sink share the first token's softmax
    q = torch.zeros(3, 1, 2, dtype=F)
    kk = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]], [[1.0, 1.0]]], dtype=F)
    out = pv.window_sink_attention(q, kk, kk, 1.0, 2, torch.zeros(1, dtype=F))
    assert out[0, 0].tolist() == [0.5, 0.0] and torch.allclose(out[2, 0], torch.tensor([1.0 / 3, 2.0 / 3], dtype=F))
    # the router: groups judged by the sum of their two best corrected scores; weights without the correction
    z = torch.tensor([3.0, -3.0, 1.0, 1.2, 0.0, 0.0], dtype=F)
    ids, wts = pv.route(z, torch.zeros(6, dtype=F), 2, 3, 1)
    assert ids == [3, 2] and abs(float(wts[0]) - 1 / (1 + math.exp(-1.2))) < 1e-12       # group 1 (1.50) beats group 0 (1.00)
    ids, _ = pv.route(z, torch.tensor([0.6, 0, 0, 0, 0, 0], dtype=F), 2, 3, 1)
    assert ids == [0, 1]                                                              # the correction lifts group 0 over it
    ids, wts = pv.route(z, torch.full((6,), -5.0, dtype=F), 2, 3, 1)
    assert ids == [3, 2] and float(wts[1]) > 0.7                                       # negative choice scores, the same choice
    # rotation by halves leaves the elements behind the rotated ones alone and keeps the length of each pair
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0]]], dtype=F)
    y = pv.rotate_halves(x, 3, {"base": 10.0, "dims": 4})
    assert float(y[0, 0, 4]) == 5.0 and abs(float(y[0, 0, 0] ** 2 + y[0, 0, 2] ** 2) - 10.0) < 1e-12
    assert abs(float(y[0, 0, 0]) - (math.cos(3.0) - 3.0 * math.sin(3.0))) < 1e-12
