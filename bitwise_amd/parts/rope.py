"""Rotary position encoding in the rotate-half layout (src/kernels.cpp:273-289).

inv_freq[i] = 1.0f / powf(theta, float(2i)/float(hd)) (src/model.cpp:220-225) and
angle = float(pos) * inv_freq[i] are 32-bit values, as in the reference; cosine and sine of
that 32-bit angle are evaluated in double and rounded once.  The tables are built on the host
for all positions up to ``max_positions`` and read by the kernels.
"""

from __future__ import annotations

import numpy as np
import torch

from .base import PositionEncoding, register_position_encoding


@register_position_encoding("rope")
class RotaryTable(PositionEncoding):
    """params: theta, head_dim, max_positions.  No checkpoint tensors."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.theta = float(params["theta"])
        self.head_dim = int(params["head_dim"])
        self.max_positions = int(params["max_positions"])
        if self.head_dim % 2:
            raise ValueError("rotary encoding needs an even head size")
        self.rotary_dim = self.head_dim          # whole heads are rotated
        self._cos = self._sin = None

    def _build(self) -> None:
        runtime = self.rt
        half = self.head_dim // 2
        i = np.arange(half, dtype=np.float32)
        expo = (np.float32(2.0) * i) / np.float32(self.head_dim)
        inv_freq = (np.float32(1.0) / np.power(np.float32(self.theta), expo, dtype=np.float32)).astype(np.float32)
        pos = np.arange(self.max_positions, dtype=np.float32)[:, None]
        angle = (pos * inv_freq[None, :]).astype(np.float32).astype(np.float64)
        self._cos = torch.from_numpy(np.cos(angle).astype(np.float32)).to(runtime.device).contiguous()
        self._sin = torch.from_numpy(np.sin(angle).astype(np.float32)).to(runtime.device).contiguous()

    def tables(self):
        if self._cos is None:
            self._build()
        return self._cos, self._sin

    @classmethod
    def shared(cls, params, runtime) -> "RotaryTable":
        key = ("rope", float(params["theta"]), int(params["head_dim"]), int(params["max_positions"]))
        return runtime.shared(key, lambda: cls(params, runtime))


@register_position_encoding("rope_pairs")
class PairRotaryTable(PositionEncoding):
    """Rotary angles for mixers that rotate neighbouring pairs (2i, 2i+1) of a head's first ``dims`` elements:
    angle = position * f_i, f_i = base^(-2i/dims), optionally stretched band by band.

    params: base, dims, max_positions; optional ``scaling`` = {factor, low, high, original}: with the wavelength
    l = 2 pi / f, a frequency stays where l < original / high, becomes f / factor where l > original / low, and in
    between is (1 - s) f / factor + s f with s = (original / l - low) / (high - low).
    Frequencies and angles are computed in double precision on the host and the cosines and sines rounded once to
    32-bit.  No checkpoint tensors.  The tables are what the base class promises, [positions, dims / 2]; which
    elements a column pairs is the mixer's business (``layout``)."""

    graph_safe = True
    launches_through_ops = True
    layout = "pairs"

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.base = float(params["base"])
        self.rotary_dim = int(params["dims"])
        self.max_positions = int(params["max_positions"])
        self.scaling = dict(params["scaling"]) if params.get("scaling") else None
        if self.rotary_dim % 2 or self.rotary_dim < 0:
            raise ValueError("rotary encoding needs an even number of rotated elements")
        if self.scaling is not None:
            missing = [k for k in ("factor", "low", "high", "original") if k not in self.scaling]
            if missing:
                raise ValueError(f"rope_pairs: scaling lacks {missing}")
            if float(self.scaling["high"]) == float(self.scaling["low"]):
                raise ValueError("rope_pairs: scaling needs high != low")
        self._cos = self._sin = None

    def frequencies(self) -> np.ndarray:
        half = self.rotary_dim // 2
        f = np.power(np.float64(self.base), -2.0 * np.arange(half, dtype=np.float64) / max(self.rotary_dim, 1))
        sc = self.scaling
        if sc is None:
            return f
        factor, low, high, orig = (float(sc[k]) for k in ("factor", "low", "high", "original"))
        wavelength = 2.0 * np.pi / f
        blend = (orig / wavelength - low) / (high - low)
        mixed = (1.0 - blend) * f / factor + blend * f
        return np.where(wavelength < orig / high, f, np.where(wavelength > orig / low, f / factor, mixed))

    def _build(self) -> None:
        angle = np.arange(self.max_positions, dtype=np.float64)[:, None] * self.frequencies()[None, :]
        self._cos = torch.from_numpy(np.cos(angle).astype(np.float32)).to(self.rt.device).contiguous()
        self._sin = torch.from_numpy(np.sin(angle).astype(np.float32)).to(self.rt.device).contiguous()

    def tables(self):
        if self._cos is None:
            self._build()
        return self._cos, self._sin

    @classmethod
    def shared(cls, params, runtime) -> "PairRotaryTable":
        sc = params.get("scaling")
        key = ("rope_pairs", float(params["base"]), int(params["dims"]), int(params["max_positions"]),
               None if not sc else tuple(sorted((k, float(v)) for k, v in sc.items())))
        return runtime.shared(key, lambda: cls(params, runtime))


@register_position_encoding("rope_halves")
class HalfRotaryTable(PositionEncoding):
    """Rotary angles for mixers that rotate element i of a head's first ``dims`` elements together with element
    i + dims/2 (the rotate-half layout), the rest of the head passing unchanged: angle = position * f_i,
    f_i = base^(-2i/dims), optionally stretched along a ramp over the pair index.

    params: base, dims, max_positions; optional ``scaling`` = {factor, original, fast, slow}: with
    index(t) = dims * ln(original / (2 pi t)) / (2 ln base), the pair index at which a frequency makes t turns over
    ``original`` positions, lo = max(floor(index(fast)), 0) and hi = min(ceil(index(slow)), dims - 1), a pair's
    frequency is f_i (1 - r_i) + f_i / factor * r_i with r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), and both
    cosines and sines are multiplied by 0.1 ln(factor) + 1.
    Frequencies and angles are computed in double precision on the host and the (scaled) cosines and sines rounded once
    to 32-bit.  No checkpoint tensors.  The tables are [positions, dims / 2]."""

    graph_safe = True
    launches_through_ops = True
    layout = "halves"

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.base = float(params["base"])
        self.rotary_dim = int(params["dims"])
        self.max_positions = int(params["max_positions"])
        self.scaling = dict(params["scaling"]) if params.get("scaling") else None
        if self.rotary_dim % 2 or self.rotary_dim < 0:
            raise ValueError("rotary encoding needs an even number of rotated elements")
        if self.scaling is not None:
            missing = [k for k in ("factor", "original", "fast", "slow") if k not in self.scaling]
            if missing:
                raise ValueError(f"rope_halves: scaling lacks {missing}")
            if not float(self.scaling["factor"]) > 0 or not min(float(self.scaling["fast"]), float(self.scaling["slow"])) > 0:
                raise ValueError("rope_halves: scaling needs positive factor, fast and slow")
        self._cos = self._sin = None

    def frequencies(self) -> np.ndarray:
        dims, half = self.rotary_dim, self.rotary_dim // 2
        idx = np.arange(half, dtype=np.float64)
        f = np.power(np.float64(self.base), -2.0 * idx / max(dims, 1))
        sc = self.scaling
        if sc is None:
            return f
        factor, orig = float(sc["factor"]), float(sc["original"])

        def index_of(turns: float) -> float:
            return dims * np.log(orig / (2.0 * np.pi * turns)) / (2.0 * np.log(self.base))

        lo = max(np.floor(index_of(float(sc["fast"]))), 0.0)
        hi = min(np.ceil(index_of(float(sc["slow"]))), dims - 1.0)
        ramp = np.clip((idx - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        return f / factor * ramp + f * (1.0 - ramp)

    def magnitude(self) -> float:
        return 1.0 if self.scaling is None else 0.1 * float(np.log(float(self.scaling["factor"]))) + 1.0

    def _build(self) -> None:
        angle = np.arange(self.max_positions, dtype=np.float64)[:, None] * self.frequencies()[None, :]
        mag = self.magnitude()
        self._cos = torch.from_numpy((np.cos(angle) * mag).astype(np.float32)).to(self.rt.device).contiguous()
        self._sin = torch.from_numpy((np.sin(angle) * mag).astype(np.float32)).to(self.rt.device).contiguous()

    def tables(self):
        if self._cos is None:
            self._build()
        return self._cos, self._sin

    @classmethod
    def shared(cls, params, runtime) -> "HalfRotaryTable":
        sc = params.get("scaling")
        key = ("rope_halves", float(params["base"]), int(params["dims"]), int(params["max_positions"]),
               None if not sc else tuple(sorted((k, float(v)) for k, v in sc.items())))
        return runtime.shared(key, lambda: cls(params, runtime))
