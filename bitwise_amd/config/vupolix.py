"""Typed configuration of the Vupolix decoder, read from the keys of its config.json.

Keys: ``architecture`` (the name), ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` (the weight of a sublayer's normed
output on its way into the stream), ``logit_scale``, ``loop`` = {start, stop, times} or absent (layers start .. stop-1 run
``times`` times in a row), and ``layers``: a list whose entries give ``type`` (the mixer: "wkv" or "parallel"), ``mixer``
(its sizes and constants) and ``mlp`` (the feed-forward, or null for a layer without one).  Mixer keys:

* wkv: heads, dim; ``rank``, the inner size of the decay's projection, is the rows of the tensor ``l<i>.mix.w1`` and is
  filled in from the checkpoint (``sizes_from_tensors``) if config.json does not carry it
* parallel: left = {heads, kv_heads, dim, vdim, scale, mask = {size}, rot = {base, dims, scaling = {factor, original, fast,
  slow} or absent}} and right = {heads, dim, vdim, decay (a number per head), rot = {base, dims, scaling or absent}}

mlp: {"kind": "moe", "expert": {ff}, "router": {experts, top, groups = {count, keep} or absent}, "shared": {ff} or absent}.

Optional keys with defaults that a checkpoint's config.json need not carry: ``max_positions`` (the length of the
rotary tables and the longest request), ``bos_token_id``, ``eos_token_id``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from .llama import ConfigError

ARCHITECTURE = "Vupolix"
MIXER_KEYS = {
    "wkv": ("heads", "dim"),
    "parallel": ("left", "right"),
}
LEFT_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot")
RIGHT_KEYS = ("heads", "dim", "vdim", "decay", "rot")
DEFAULT_MAX_POSITIONS = 1 << 16


def _positive_int(d: Mapping[str, Any], key: str, where: str) -> int:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or v < 1:
        raise ConfigError(f"config.json: {where} needs a positive integer '{key}', got {v!r}")
    return v


def _check_rot(rot: Any, dim: int, where: str) -> None:
    if not isinstance(rot, Mapping) or "base" not in rot or "dims" not in rot:
        raise ConfigError(f"config.json: {where} needs rot = {{base, dims}}")
    if isinstance(rot["dims"], bool) or not isinstance(rot["dims"], int) or rot["dims"] % 2 or not 0 <= rot["dims"] <= dim:
        raise ConfigError(f"config.json: {where}: rot.dims must be even and at most dim")
    if not float(rot["base"]) > 1.0:
        raise ConfigError(f"config.json: {where}: rot.base must be larger than 1")
    sc = rot.get("scaling")
    if sc is not None and (not isinstance(sc, Mapping) or any(k not in sc for k in ("factor", "original", "fast", "slow"))):
        raise ConfigError(f"config.json: {where}: rot.scaling needs factor, original, fast and slow")


@dataclass(frozen=True)
class VupolixLayer:
    type: str
    mixer: Mapping[str, Any]
    mlp: Optional[Mapping[str, Any]]          # None: the layer has no feed-forward


@dataclass(frozen=True)
class VupolixConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    residual_mult: float
    logit_scale: float
    loop: Tuple[int, int, int]                # (start, stop, times); (0, 0, 1): nothing is repeated
    layers: Tuple[VupolixLayer, ...]
    max_positions: int
    bos_token_id: int
    eos_token_id: int

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "VupolixConfig":
        name = d.get("architecture")
        if not isinstance(name, str):
            raise ConfigError("config.json lacks 'architecture': name")
        norm = d.get("norm")
        if not isinstance(norm, Mapping) or "eps" not in norm:
            raise ConfigError("config.json lacks 'norm': {'eps': ...}")
        for key in ("residual_mult", "logit_scale"):
            if key not in d or isinstance(d[key], bool) or not isinstance(d[key], (int, float)):
                raise ConfigError(f"config.json lacks a number '{key}'")
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json lacks a non-empty list 'layers'")
        layers: List[VupolixLayer] = []
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
            if kind == "wkv":
                for k in ("heads", "dim"):
                    _positive_int(mixer, k, where)
                if "rank" in mixer:
                    _positive_int(mixer, "rank", where)
            else:
                left, right = mixer["left"], mixer["right"]
                for side, keys, what in ((left, LEFT_KEYS, "left"), (right, RIGHT_KEYS, "right")):
                    if not isinstance(side, Mapping) or any(k not in side for k in keys):
                        raise ConfigError(f"config.json: {where}: mixer.{what} needs {list(keys)}")
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    _positive_int(left, k, where + " left")
                if left["heads"] % left["kv_heads"]:
                    raise ConfigError(f"config.json: {where} left: heads must be a multiple of kv_heads")
                if left["vdim"] != left["dim"]:
                    raise ConfigError(f"config.json: {where} left: the values are the keys, so vdim must equal dim")
                if not float(left["scale"]) > 0:
                    raise ConfigError(f"config.json: {where} left: scale must be positive")
                if not isinstance(left["mask"], Mapping):
                    raise ConfigError(f"config.json: {where} left: mask = {{size}}")
                _positive_int(left["mask"], "size", where + " left.mask")
                _check_rot(left["rot"], left["dim"], where + " left")
                for k in ("heads", "dim", "vdim"):
                    _positive_int(right, k, where + " right")
                decay = right["decay"]
                if not isinstance(decay, (list, tuple)) or len(decay) != right["heads"] or any(
                        isinstance(x, bool) or not isinstance(x, (int, float)) or not 0.0 <= float(x) <= 1.0 for x in decay):
                    raise ConfigError(f"config.json: {where} right: decay must give a number in [0, 1] per head")
                _check_rot(right["rot"], right["dim"], where + " right")
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") != "moe":
                    raise ConfigError(f"config.json: {where} has an mlp of kind {mlp.get('kind') if isinstance(mlp, Mapping) else mlp!r}; known: moe")
                ex, ro = mlp.get("expert"), mlp.get("router")
                if not isinstance(ex, Mapping) or not isinstance(ro, Mapping):
                    raise ConfigError(f"config.json: {where} mlp needs expert = {{ff}} and router = {{experts, top}}")
                _positive_int(ex, "ff", where + " mlp.expert")
                experts, top = _positive_int(ro, "experts", where + " mlp.router"), _positive_int(ro, "top", where + " mlp.router")
                groups = ro.get("groups")
                count, keep = 1, 1
                if groups is not None:
                    count, keep = _positive_int(groups, "count", where + " mlp.router.groups"), _positive_int(groups, "keep", where + " mlp.router.groups")
                if experts % count or keep > count or top > keep * (experts // count):
                    raise ConfigError(f"config.json: {where}: {top} of {experts} experts in {count} groups of which {keep} are kept does not work out")
                if mlp.get("shared") is not None:
                    if not isinstance(mlp["shared"], Mapping):
                        raise ConfigError(f"config.json: {where} mlp.shared = {{ff}}")
                    _positive_int(mlp["shared"], "ff", where + " mlp.shared")
            layers.append(VupolixLayer(kind, copy.deepcopy(dict(mixer)), None if mlp is None else copy.deepcopy(dict(mlp))))
        loop = d.get("loop")
        span = (0, 0, 1)
        if loop is not None:
            if not isinstance(loop, Mapping) or any(isinstance(loop.get(k), bool) or not isinstance(loop.get(k), int) for k in ("start", "stop", "times")):
                raise ConfigError("config.json: loop = {start, stop, times}, three integers")
            span = (int(loop["start"]), int(loop["stop"]), int(loop["times"]))
            if not 0 <= span[0] <= span[1] <= len(layers) or span[2] < 1:
                raise ConfigError(f"config.json: loop {dict(loop)} does not fit {len(layers)} layers")
        eos, bos = d.get("eos_token_id", -1), d.get("bos_token_id", -1)
        return cls(architecture=name, vocab=_positive_int(d, "vocab", "the model"), width=_positive_int(d, "width", "the model"),
                   eps=float(norm["eps"]), residual_mult=float(d["residual_mult"]), logit_scale=float(d["logit_scale"]), loop=span,
                   layers=tuple(layers), max_positions=int(d.get("max_positions", DEFAULT_MAX_POSITIONS)),
                   bos_token_id=-1 if bos is None else int(bos), eos_token_id=-1 if eos is None else int(eos))

    def to_dict(self) -> Dict[str, Any]:
        return {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
            "residual_mult": self.residual_mult, "logit_scale": self.logit_scale,
            "loop": {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]},
            "layers": [{"type": l.type, "mixer": copy.deepcopy(dict(l.mixer)),
                        "mlp": None if l.mlp is None else copy.deepcopy(dict(l.mlp))} for l in self.layers],
            "max_positions": self.max_positions, "bos_token_id": self.bos_token_id, "eos_token_id": self.eos_token_id,
        }

    def layer_runs(self) -> List[Tuple[int, bool]]:
        """(layer, whether a further pass of the repeated layers starts with it) in the order the layers run."""
        start, stop, times = self.loop
        runs = [(i, False) for i in range(start)]
        for p in range(times):
            runs += [(i, p > 0 and i == start) for i in range(start, stop)]
        return runs + [(i, False) for i in range(stop, len(self.layers))]


def sizes_from_tensors(config: Mapping[str, Any], shapes: Mapping[str, Tuple[int, ...]]) -> Dict[str, Any]:
    """The configuration with the sizes that only the checkpoint's tensor shapes give filled in: a wkv layer's ``rank``."""
    out = copy.deepcopy(dict(config))
    for i, entry in enumerate(out.get("layers") or []):
        if isinstance(entry, dict) and entry.get("type") == "wkv" and isinstance(entry.get("mixer"), dict):
            shape = shapes.get(f"l{i}.mix.w1")
            if "rank" not in entry["mixer"] and shape is not None and len(shape) == 2:
                entry["mixer"]["rank"] = int(shape[0])
    return out
