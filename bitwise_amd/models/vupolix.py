"""The Vupolix decoder as a ModelSpec: an embedding that is normed; layers x += m norm1b(mixer(norm1(x))); x += m
norm2b(ff(norm2(x))) (a norm in front of each sublayer and one behind it, m the residual weight) whose mixers are, layer
by layer, RWKV-style time mixing (the token shift rides in norm1, which delivers five mixes) or two mixers side by side
(windowed attention whose values are its keys, with a learned sink and a gate per head, beside retention) whose normed
outputs are averaged; feed-forwards of routed experts with sigmoid scores, a correction for the choice and a shared
expert; a span of layers that runs several times, each pass with caches and state of its own and the embedding's
output added in front of every pass but the first; a final norm and an untied head whose logits are scaled.
Layer i's tensors start with ``l<i>.``: norm1, norm1b, norm2, norm2b, mix.*, mlp.*; the rest are ``embed``,
``embed.norm``, ``final.norm`` and ``head``."""

from __future__ import annotations

from ..config.vupolix import VupolixConfig
from ..parts.base import LayerCall, LayerSpec, ModelSpec, PartSpec

# A small configuration for simulations and smoke runs: sizes that are all different, a layer without feed-forward, the
# middle layers run three times, fewer key heads than query heads, a partly rotated head, values wider than keys in
# the retention branch, experts in three groups and without groups.
TINY_VUPOLIX = {
    "architecture": "Vupolix", "vocab": 89, "width": 40, "norm": {"eps": 1e-5}, "residual_mult": 0.4, "logit_scale": 0.7,
    "max_positions": 512, "eos_token_id": 2, "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "parallel",
         "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 16, "scale": 0.3, "mask": {"size": 24},
                            "rot": {"base": 1000.0, "dims": 8, "scaling": {"factor": 3.0, "original": 64, "fast": 8.0, "slow": 2.0}}},
                   "right": {"heads": 2, "dim": 8, "vdim": 24, "decay": [0.9, 0.97], "rot": {"base": 500.0, "dims": 6}}},
         "mlp": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}},
                 "shared": {"ff": 24}}},
        {"type": "wkv", "mixer": {"heads": 3, "dim": 8, "rank": 5}, "mlp": None},
        {"type": "parallel",
         "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 24, "vdim": 24, "scale": 0.2, "mask": {"size": 7},
                            "rot": {"base": 100.0, "dims": 24}},
                   "right": {"heads": 3, "dim": 16, "vdim": 8, "decay": [0.8, 0.95, 0.99], "rot": {"base": 300.0, "dims": 16}}},
         "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 4, "top": 3}}},
        {"type": "wkv", "mixer": {"heads": 2, "dim": 16, "rank": 3},
         "mlp": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 8, "top": 2, "groups": {"count": 2, "keep": 1}},
                 "shared": {"ff": 8}}},
    ],
}

WKV_MIXES = ("r", "k", "v", "g", "w")


def vupolix_spec(cfg: VupolixConfig) -> ModelSpec:
    layers = []
    for i, layer in enumerate(cfg.layers):
        pre = f"l{i}."
        m = dict(layer.mixer)
        norm = lambda tensor, **more: PartSpec("rmsnorm", dict({"width": cfg.width, "eps": cfg.eps, "tensor": tensor}, **more), pre)
        if layer.type == "wkv":
            if "rank" not in m:
                raise ValueError(f"layer {i}: the decay projection's inner size is not known (the rows of {pre}mix.w1)")
            mixer = PartSpec("wkv", {"width": cfg.width, "heads": int(m["heads"]), "dim": int(m["dim"]), "eps": cfg.eps,
                                     "rank": int(m["rank"]), "inputs": WKV_MIXES}, pre + "mix.")
            mixer_norm = PartSpec("rmsnorm_shift", {"width": cfg.width, "eps": cfg.eps, "tensor": "norm1",
                                                    "mix_tensors": [f"mix.mu.{s}" for s in WKV_MIXES]}, pre)
        else:
            left, right = dict(m["left"]), dict(m["right"])
            lrot, rrot = dict(left["rot"]), dict(right["rot"])
            attention = PartSpec("gated_attention", {
                "width": cfg.width, "heads": int(left["heads"]), "kv_heads": int(left["kv_heads"]), "dim": int(left["dim"]),
                "vdim": int(left["vdim"]), "scale": float(left["scale"]), "eps": cfg.eps, "conv": 0, "qk_norm": False,
                "sink": "learned", "gate": "head", "values": "keys", "shared_kv": False, "window": int(left["mask"]["size"]),
                "position": PartSpec("rope_halves", {"base": float(lrot["base"]), "dims": int(lrot["dims"]),
                                                     "scaling": lrot.get("scaling"), "max_positions": cfg.max_positions})})
            retention = PartSpec("retention", {
                "width": cfg.width, "heads": int(right["heads"]), "dim": int(right["dim"]), "vdim": int(right["vdim"]),
                "eps": cfg.eps, "decay": [float(x) for x in right["decay"]],
                "position": PartSpec("rope_halves", {"base": float(rrot["base"]), "dims": int(rrot["dims"]),
                                                     "scaling": rrot.get("scaling"), "max_positions": cfg.max_positions})})
            mixer = PartSpec("side_by_side", {"width": cfg.width, "eps": cfg.eps,
                                              "branches": [("left", attention), ("right", retention)]}, pre + "mix.")
            mixer_norm = norm("norm1")
        parts = {"mixer_norm": mixer_norm, "mixer": mixer, "mixer_post_norm": norm("norm1b", scale=cfg.residual_mult)}
        mlp = layer.mlp
        if mlp is not None:
            ro = mlp["router"]
            groups = ro.get("groups") or {"count": 1, "keep": 1}
            parts["ffn_norm"] = norm("norm2")
            parts["ffn_post_norm"] = norm("norm2b", scale=cfg.residual_mult)
            parts["feed_forward"] = PartSpec("moe", {
                "width": cfg.width, "experts": int(ro["experts"]), "top": int(ro["top"]), "groups": int(groups["count"]),
                "keep": int(groups["keep"]), "ff": int(mlp["expert"]["ff"]), "limit": None, "alpha": 1.0,
                "score": "sigmoid", "correction": True, "group_best": 2,
                "shared": None if mlp.get("shared") is None else {"ff": int(mlp["shared"]["ff"]), "gated": False}}, pre + "mlp.")
        layers.append(LayerSpec("sandwich", parts))
    # every run of a layer has a cache and state of its own
    schedule = [LayerCall(layer=i, cache=n, adds_embedding=again) for n, (i, again) in enumerate(cfg.layer_runs())]
    return ModelSpec(
        architecture=cfg.architecture,
        vocab_size=cfg.vocab,
        width=cfg.width,
        embedding=PartSpec("embedding", {"vocab": cfg.vocab, "width": cfg.width, "tensor": "embed",
                                         "norm": {"tensor": "embed.norm", "eps": cfg.eps}}, ""),
        layers=layers,
        schedule=schedule,
        final_norm=PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps, "tensor": "norm"}, "final."),
        lm_head=PartSpec("lm_head", {"vocab": cfg.vocab, "width": cfg.width, "tied": False, "tensor": "head",
                                     "scale": cfg.logit_scale}, ""),
        max_positions=cfg.max_positions,
        bos_token_id=cfg.bos_token_id,
        eos_token_id=cfg.eos_token_id,
    )
