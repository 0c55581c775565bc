"""The Kikarax decoder as a ModelSpec: an embedding that adds a hashed token-pair row and a learned position row to the
scaled token row; pre-norm layers x += mixer(norm1(x)); x += ff(norm2(x)) whose mixers are gated attention without
rotation (queries and keys normed over their whole projections, soft-capped scores, chunks of positions, values mixed
with the first such layer's) and whose feed-forwards are a clamped gated unit or routed experts beside a gated shared
expert; a final norm and a head tied to the token table, its logits scaled.  Layer i's tensors start with ``l<i>.``:
norm1, norm2, mix.*, mlp.*; the rest are ``embed``, ``bigram``, ``pos`` and ``final.norm``."""

from __future__ import annotations

from ..config.kikarax import KikaraxConfig
from ..parts.base import LayerCall, LayerSpec, ModelSpec, PartSpec

# A small configuration for simulations and smoke runs: sizes that are all different, a layer without feed-forward, a
# layer without chunks, cap and value mixing, chunks of different sizes, fewer key heads than query heads.
TINY_KIKARAX = {
    "architecture": "Kikarax", "vocab": 101, "width": 48, "norm": {"eps": 1e-5}, "logit_scale": 0.5, "max_positions": 512,
    "eos_token_id": 2,
    "embedding": {"scale": 3.0, "bigram": {"buckets": 37, "mul_prev": 11, "mul_cur": 5}},
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 0.3, "softcap": 10.0, "mask": {"size": 24}, "v_mix": True},
         "mlp": {"kind": "dense", "ff": 40, "limit": 1.5}},
        {"type": "attention",
         "mixer": {"heads": 2, "kv_heads": 1, "dim": 24, "vdim": 16, "scale": 0.25},
         "mlp": None},
        {"type": "attention",
         "mixer": {"heads": 6, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.4, "softcap": 20.0, "mask": {"size": 40}, "v_mix": True},
         "mlp": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 6, "top": 2, "scale": 1.5}, "shared": {"ff": 24}}},
    ],
}


def kikarax_spec(cfg: KikaraxConfig) -> ModelSpec:
    layers, schedule = [], []
    source_seen = False
    for i, layer in enumerate(cfg.layers):
        pre = f"l{i}."
        m = dict(layer.mixer)
        v_mix = None
        if m.get("v_mix"):
            v_mix = "mix" if source_seen else "source"
            source_seen = True
        mixer = PartSpec("gated_attention", {
            "width": cfg.width, "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]),
            "vdim": int(m["vdim"]), "scale": float(m["scale"]), "eps": cfg.eps, "conv": 0, "qk_norm": "whole", "sink": None,
            "gate": True, "shared_kv": False, "window": None, "position": None,
            "softcap": None if m.get("softcap") is None else float(m["softcap"]),
            "chunk": None if m.get("mask") is None else int(m["mask"]["size"]), "v_mix": v_mix}, pre + "mix.")
        schedule.append(LayerCall(layer=i, cache=i))
        parts = {
            "mixer_norm": PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps, "tensor": "norm1"}, pre),
            "mixer": mixer,
        }
        mlp = layer.mlp
        if mlp is not None:
            parts["ffn_norm"] = PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps, "tensor": "norm2"}, pre)
            if mlp["kind"] == "dense":
                parts["feed_forward"] = PartSpec("clamped_glu", {"width": cfg.width, "inter": int(mlp["ff"]), "limit": float(mlp["limit"]),
                                                                 "alpha": 1.702, "names": ("gate", "up", "down")}, pre + "mlp.")
            else:
                ro = mlp["router"]
                parts["feed_forward"] = PartSpec("moe", {
                    "width": cfg.width, "experts": int(ro["experts"]), "top": int(ro["top"]), "groups": 1, "keep": 1,
                    "ff": int(mlp["expert"]["ff"]), "limit": None, "alpha": 1.0, "weight_scale": float(ro.get("scale") or 1.0),
                    "shared": None if mlp.get("shared") is None else {"ff": int(mlp["shared"]["ff"])}}, pre + "mlp.")
        layers.append(LayerSpec("prenorm", parts))
    pairs = None if cfg.bigram is None else dict(cfg.bigram, tensor="bigram")
    return ModelSpec(
        architecture=cfg.architecture,
        vocab_size=cfg.vocab,
        width=cfg.width,
        embedding=PartSpec("embedding_sum", {"vocab": cfg.vocab, "width": cfg.width, "tensor": "embed", "scale": cfg.embedding_scale,
                                             "pairs": pairs, "positions": {"tensor": "pos", "count": cfg.max_positions}}, ""),
        layers=layers,
        schedule=schedule,
        final_norm=PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.eps, "tensor": "norm"}, "final."),
        lm_head=PartSpec("lm_head", {"vocab": cfg.vocab, "width": cfg.width, "tied": True, "scale": cfg.logit_scale}, ""),
        max_positions=cfg.max_positions,
        bos_token_id=cfg.bos_token_id,
        eos_token_id=cfg.eos_token_id,
    )
