"""RMSNorm: y = (x * 1/sqrt(mean(x^2) + eps)) * weight (src/kernels.cpp:264-271), with a weight that may be
stored as its distance from 1, and the variant that mixes the previous token's normed row into the output."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from .base import Norm, StateSpec, TensorSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """params: width, eps; optional ``offset`` (the stored weight w is applied as offset + w; 0 by default, 1 for a
    weight kept as its distance from 1), ``tensor`` (the weight's name behind the prefix, "weight" by default) and
    ``scale`` (1 by default): where the norm sits behind a sublayer, the stream receives scale * norm(y).
    The sum of squares, the root and both products are 32-bit; the output has the mode's activation dtype."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.width = int(params["width"])
        self.eps = float(params["eps"])
        self.offset = float(params.get("offset", 0.0))
        self.tensor = str(params.get("tensor", "weight"))
        self.scale = float(params.get("scale", 1.0))
        self.weight = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.width,), "around_zero" if self.offset else "norm")}

    def _applied(self, w: torch.Tensor) -> torch.Tensor:
        w = w.to(self.rt.device)
        if self.offset:
            w = w.float() + self.offset         # one 32-bit addition; the kernels multiply by the sum
        return w.contiguous()

    def bind(self, tensors) -> None:
        self.weight = self._applied(tensors[self.tensor])

    def weight_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def forward(self, ctx, x: torch.Tensor, out_name: str = "normed", rows: int | None = None) -> torch.Tensor:
        rows = ctx.rows if rows is None else rows
        out = ctx.ws.buffer(out_name, self.width, self.rt.act_dtype)
        ops.rmsnorm(x, self.weight, out, rows, self.eps)
        return out

    def add_normed(self, ctx, y: torch.Tensor, x: torch.Tensor, rounded: Optional[torch.Tensor] = None) -> None:
        """x += scale * (y / sqrt(mean(y^2) + eps) * weight), one kernel, all 32-bit; ``rounded``: the new x once more, in bfloat16."""
        ops.norm_add(y, self.weight, x, ctx.rows, self.eps, rounded, scale=self.scale)


@register_norm("rmsnorm_shift")
class ShiftedRMSNorm(RMSNorm):
    """RMSNorm followed by a token shift: with h the normed rows, the output is h_t + (h_{t-1} - h_t) * mix, element by
    element, h_{t-1} the same request's normed row of the token before (zeros before its first token).  The last normed
    row of every request is per-request state, so that the next step's first row finds it.  params as RMSNorm, plus
    ``mix_tensor`` (the name of the mixing weights [width], "shift" by default) or ``mix_tensors`` (several names: the
    output then holds one shifted copy of the row per mixing vector, side by side, [rows, n * width], for a mixer whose
    projections each read a mix of their own).  Norm and shift are one kernel, all 32-bit."""

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        many = params.get("mix_tensors")
        self.mix_tensors = [str(n) for n in many] if many else [str(params.get("mix_tensor", "shift"))]
        self.mix: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        out = super().tensors()
        for name in self.mix_tensors:
            out[name] = TensorSpec((self.width,), "unit_interval")
        return out

    def bind(self, tensors) -> None:
        self.weight = self._applied(tensors[self.tensor]).float().contiguous()
        self.mix = torch.stack([tensors[n].to(self.rt.device).float() for n in self.mix_tensors]).contiguous()

    def weight_bytes(self) -> int:
        return super().weight_bytes() + self.mix.numel() * 4

    def state_spec(self) -> StateSpec:
        return StateSpec((self.width,), "float32")

    def forward(self, ctx, x: torch.Tensor, out_name: str = "normed_shifted", rows: int | None = None,
                state: Optional[torch.Tensor] = None) -> torch.Tensor:
        if state is None:
            raise ValueError("rmsnorm_shift: the block must hand over the call's state (a row per slot)")
        rows = ctx.rows if rows is None else rows
        out = ctx.ws.buffer(out_name, len(self.mix_tensors) * self.width, self.rt.act_dtype)
        ops.norm_shift(x, self.weight, self.mix, state, ctx.positions, ctx.row_seq, ctx.seq_rows, ctx.slots, out, rows, self.eps)
        return out
