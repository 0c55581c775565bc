"""Typed configuration of the Kikarax decoder, read from the keys of its config.json.

Keys: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps``, ``logit_scale``, ``max_positions`` (rows of the
learned position table), ``embedding`` = {scale, bigram = {buckets, mul_prev, mul_cur} or absent}, and ``layers``: a list
whose entries give ``type`` (the mixer: "attention"), ``mixer`` (its sizes and constants) and ``mlp`` (the feed-forward,
or null for a layer without one).

* attention: heads, kv_heads, dim, vdim, scale; optional softcap, mask = {size} (chunks of that many positions), v_mix
* mlp: {"kind": "dense", ff, limit} or {"kind": "moe", "expert": {ff}, "router": {experts, top, scale}, "shared": {ff} or absent}

Optional keys with defaults that a checkpoint's config.json need not carry: ``bos_token_id``, ``eos_token_id``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .llama import ConfigError

ARCHITECTURE = "Kikarax"
MIXER_KEYS = {"attention": ("heads", "kv_heads", "dim", "vdim", "scale")}


def _positive_int(d: Mapping[str, Any], key: str, where: str) -> int:
    v = d.get(key) if isinstance(d, Mapping) else None
    if isinstance(v, bool) or not isinstance(v, int) or v < 1:
        raise ConfigError(f"config.json: {where} needs a positive integer '{key}', got {v!r}")
    return v


def _positive(d: Mapping[str, Any], key: str, where: str) -> float:
    v = d.get(key) if isinstance(d, Mapping) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not float(v) > 0:
        raise ConfigError(f"config.json: {where} needs a positive number '{key}', got {v!r}")
    return float(v)


@dataclass(frozen=True)
class KikaraxLayer:
    type: str
    mixer: Mapping[str, Any]
    mlp: Optional[Mapping[str, Any]]          # None: the layer has no feed-forward


@dataclass(frozen=True)
class KikaraxConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    logit_scale: float
    embedding_scale: float
    bigram: Optional[Mapping[str, int]]       # {buckets, mul_prev, mul_cur}
    layers: Tuple[KikaraxLayer, ...]
    max_positions: int
    bos_token_id: int
    eos_token_id: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "KikaraxConfig":
        name = d.get("architecture")
        if not isinstance(name, str):
            raise ConfigError("config.json lacks 'architecture': name")
        norm = d.get("norm")
        if not isinstance(norm, Mapping) or "eps" not in norm:
            raise ConfigError("config.json lacks 'norm': {'eps': ...}")
        emb = d.get("embedding")
        if not isinstance(emb, Mapping) or "scale" not in emb:
            raise ConfigError("config.json lacks 'embedding': {'scale': ...}")
        bigram = emb.get("bigram")
        if bigram is not None:
            _positive_int(bigram, "buckets", "embedding.bigram")
            for k in ("mul_prev", "mul_cur"):
                v = bigram.get(k)
                if isinstance(v, bool) or not isinstance(v, int) or v < 0:
                    raise ConfigError(f"config.json: embedding.bigram needs an integer '{k}' that is not negative, got {v!r}")
            bigram = {k: int(bigram[k]) for k in ("buckets", "mul_prev", "mul_cur")}
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json lacks a non-empty list 'layers'")
        layers: List[KikaraxLayer] = []
        mixed: Optional[int] = None          # kv_heads * vdim of the layers that mix values
        for i, entry in enumerate(raw_layers):
            where = f"layer {i}"
            kind = entry.get("type") if isinstance(entry, Mapping) else None
            if kind not in MIXER_KEYS:
                raise ConfigError(f"config.json: {where} has type {kind!r}; known: {sorted(MIXER_KEYS)}")
            mixer = entry.get("mixer")
            if not isinstance(mixer, Mapping):
                raise ConfigError(f"config.json: {where} lacks 'mixer'")
            missing = [k for k in MIXER_KEYS[kind] if k not in mixer]
            if missing:
                raise ConfigError(f"config.json: {where} ({kind}) lacks mixer keys {missing}")
            for k in ("heads", "kv_heads", "dim", "vdim"):
                _positive_int(mixer, k, where)
            if int(mixer["heads"]) % int(mixer["kv_heads"]):
                raise ConfigError(f"config.json: {where}: heads must be a multiple of kv_heads")
            _positive(mixer, "scale", where)
            if mixer.get("softcap") is not None:
                _positive(mixer, "softcap", where)
            if mixer.get("mask") is not None:
                _positive_int(mixer["mask"], "size", where + " mask")
            if mixer.get("v_mix"):
                here = int(mixer["kv_heads"]) * int(mixer["vdim"])
                if mixed is not None and mixed != here:
                    raise ConfigError(f"config.json: {where}: layers that mix values need values of one size (kv_heads * vdim)")
                mixed = here
            mlp = entry.get("mlp")
            if mlp is not None:
                mk = mlp.get("kind") if isinstance(mlp, Mapping) else None
                if mk == "dense":
                    _positive_int(mlp, "ff", where + " mlp")
                    _positive(mlp, "limit", where + " mlp")
                elif mk == "moe":
                    ex, ro = mlp.get("expert"), mlp.get("router")
                    _positive_int(ex, "ff", where + " mlp.expert")
                    experts, top = _positive_int(ro, "experts", where + " mlp.router"), _positive_int(ro, "top", where + " mlp.router")
                    if top > experts:
                        raise ConfigError(f"config.json: {where}: {top} of {experts} experts does not work out")
                    if ro.get("scale") is not None:
                        _positive(ro, "scale", where + " mlp.router")
                    if mlp.get("shared") is not None:
                        _positive_int(mlp["shared"], "ff", where + " mlp.shared")
                else:
                    raise ConfigError(f"config.json: {where} has an mlp of kind {mk!r}; known: dense, moe")
            layers.append(KikaraxLayer(kind, copy.deepcopy(dict(mixer)), None if mlp is None else copy.deepcopy(dict(mlp))))
        eos, bos = d.get("eos_token_id", -1), d.get("bos_token_id", -1)
        return cls(architecture=name, vocab=_positive_int(d, "vocab", "the model"), width=_positive_int(d, "width", "the model"),
                   eps=float(norm["eps"]), logit_scale=float(d.get("logit_scale", 1.0)), embedding_scale=float(emb["scale"]),
                   bigram=bigram, layers=tuple(layers), max_positions=_positive_int(d, "max_positions", "the model"),
                   bos_token_id=-1 if bos is None else int(bos), eos_token_id=-1 if eos is None else int(eos))

    def to_dict(self) -> Dict[str, Any]:
        emb: Dict[str, Any] = {"scale": self.embedding_scale}
        if self.bigram is not None:
            emb["bigram"] = dict(self.bigram)
        return {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
            "logit_scale": self.logit_scale, "embedding": emb,
            "layers": [{"type": l.type, "mixer": copy.deepcopy(dict(l.mixer)),
                        "mlp": None if l.mlp is None else copy.deepcopy(dict(l.mlp))} for l in self.layers],
            "max_positions": self.max_positions, "bos_token_id": self.bos_token_id, "eos_token_id": self.eos_token_id,
        }
