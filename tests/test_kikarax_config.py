"""The Kikarax configuration and registry on the CPU: keys read from config.json, refusals, the tensors a configuration
names, which layers keep and which mix values, the plain implementation's own mechanisms on small cases worked by hand,
and a model folder written and read back."""

import copy

import pytest
import torch

import plain_kikarax as pk
from bitwise_amd.config.kikarax import KikaraxConfig
from bitwise_amd.config.llama import ConfigError
from bitwise_amd.model import describe, model_spec, write_random_model
from bitwise_amd.models.kikarax import TINY_KIKARAX
from bitwise_amd.registry import ARCHITECTURES, architecture_of, read_model_config


def test_registry_and_round_trip():
    arch = architecture_of(TINY_KIKARAX)
    assert arch is ARCHITECTURES["Kikarax"] and arch.tiny_config is TINY_KIKARAX
    cfg = KikaraxConfig.from_dict(TINY_KIKARAX)
    again = KikaraxConfig.from_dict(cfg.to_dict())
    assert again == cfg and cfg.layers[1].mlp is None and cfg.layers[1].mixer.get("mask") is None
    assert cfg.logit_scale == 0.5 and cfg.embedding_scale == 3.0 and cfg.bigram == {"buckets": 37, "mul_prev": 11, "mul_cur": 5}


def test_tensor_names_and_parts():
    spec = model_spec(TINY_KIKARAX)
    t = describe(TINY_KIKARAX)
    assert t["embed"].shape == (101, 48) and t["bigram"].shape == (38, 48) and t["pos"].shape == (512, 48)
    assert "head" not in t and t["final.norm"].shape == (48,)
    assert t["l0.mix.q"].shape == (64, 48) and t["l0.mix.k"].shape == (32, 48) and t["l0.mix.v"].shape == (16, 48)
    assert t["l0.mix.q.norm"].shape == (64,) and t["l0.mix.k.norm"].shape == (32,) and t["l0.mix.vmix"].shape == ()
    assert t["l0.mix.g"].shape == (32, 48) and t["l0.mix.o"].shape == (48, 32)
    assert t["l0.mlp.gate"].shape == (40, 48) and t["l0.mlp.down"].shape == (48, 40)
    assert "l1.norm2" not in t and "l1.mix.vmix" not in t
    assert t["l2.mlp.router"].shape == (6, 48) and t["l2.mlp.e5.down"].shape == (48, 16) and "l2.mlp.e6.gate" not in t
    assert t["l2.mlp.shared.sg"].shape == (1, 48) and t["l2.mlp.shared.up"].shape == (24, 48)
    mix = [l.mixer.params for l in spec.layers]
    assert [m["v_mix"] for m in mix] == ["source", None, "mix"]
    assert [m["chunk"] for m in mix] == [24, None, 40] and [m["softcap"] for m in mix] == [10.0, None, 20.0]
    assert all(m["position"] is None and m["qk_norm"] == "whole" for m in mix)
    assert all(l.block == "prenorm" for l in spec.layers) and "feed_forward" not in spec.layers[1].parts
    assert spec.lm_head.params["tied"] and spec.lm_head.params["scale"] == 0.5
    assert spec.layers[2].parts["feed_forward"].params["weight_scale"] == 1.5


@pytest.mark.parametrize("change, what", [
    (lambda c: c.pop("embedding"), "embedding"),
    (lambda c: c.pop("max_positions"), "max_positions"),
    (lambda c: c["embedding"]["bigram"].update(buckets=0), "buckets"),
    (lambda c: c["layers"][0].update(type="mamba"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"].update(softcap=-1.0), "softcap"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=16), "values of one size"),
    (lambda c: c["layers"][2]["mlp"]["router"].update(top=7), "experts"),
    (lambda c: c["layers"][0]["mlp"].pop("limit"), "limit"),
    (lambda c: c["layers"][0]["mlp"].update(kind="glu"), "kind"),
])
def test_refusals(change, what):
    cfg = copy.deepcopy(TINY_KIKARAX)
    change(cfg)
    with pytest.raises(ConfigError) as e:
        KikaraxConfig.from_dict(cfg)
    assert what in str(e.value)


def test_a_model_folder_comes_back(tmp_path):
    from bitwise_amd.weights import loader
    folder = write_random_model(tmp_path / "m", TINY_KIKARAX, 5, 0.1)
    raw = read_model_config(folder)
    assert KikaraxConfig.from_dict(raw) == KikaraxConfig.from_dict(TINY_KIKARAX)
    w = loader.load_folder(folder, describe(raw))
    assert w["l2.mix.vmix"].shape == () and 0.0 < float(w["l2.mix.vmix"]) < 1.0 and w["bigram"].shape == (38, 48)


def test_the_plain_mechanisms_by_hand():
    # the pair table's rows: the first token takes the row behind the buckets, the others the hash of (before, token)
    assert pk.bigram_rows([4, 9, 9, 0], 7, 3, 5) == [7, (4 * 3 + 9 * 5) % 7, (9 * 3 + 9 * 5) % 7, (9 * 3) % 7]
    # chunks counted from position 0
    m = pk.visible(7, 3)
    assert m[2].tolist() == [True, True, True, False, False, False, False]
    assert m[3].tolist() == [False, False, False, True, False, False, False]
    assert m[6].tolist() == [False] * 6 + [True] and pk.visible(4, None)[3].tolist() == [True] * 4
    # the cap leaves small scores and bounds large ones
    s = pk.soft_cap(torch.tensor([0.01, 100.0, -100.0], dtype=pk.F), 5.0)
    assert abs(float(s[0]) - 0.01) < 1e-7 and abs(float(s[1]) - 5.0) < 1e-6 and abs(float(s[2]) + 5.0) < 1e-6
    # the router: softmax over all, the best ones' scores times the scale, not renormalized
    idx, wt = pk.route(torch.tensor([[0.0, 2.0, 1.0]], dtype=pk.F), 2, 3.0)
    e = torch.exp(torch.tensor([0.0, 2.0, 1.0], dtype=pk.F))
    assert idx.tolist() == [[1, 2]] and torch.allclose(wt[0], 3.0 * e[[1, 2]] / e.sum())
    # value mixing
    v = pk.mix_values(torch.tensor([2.0], dtype=pk.F), torch.tensor([10.0], dtype=pk.F), torch.tensor(0.25, dtype=pk.F))
    assert float(v) == 0.75 * 2.0 + 0.25 * 10.0
    # the clamped unit where both clamps bite: g = min(5, 2) = 2, u = clamp(-9, -2, 2) = -2: 2 sigmoid(3.404) (-1)
    w = {"gate": torch.tensor([[5.0]], dtype=pk.F), "up": torch.tensor([[-9.0]], dtype=pk.F), "down": torch.tensor([[1.0]], dtype=pk.F)}
    y = pk.dense_ff({"limit": 2.0}, w, "", torch.tensor([[1.0]], dtype=pk.F))
    assert abs(float(y) + 2.0 / (1.0 + torch.exp(torch.tensor(-3.404, dtype=pk.F)))) < 1e-12
