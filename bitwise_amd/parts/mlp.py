"""Dense gated feed-forward (src/model.cpp:301-305, src/kernels.cpp:291-298):
one stacked product [gate; up], h = act(g) * u, down projection added into the residual stream.
SwiGLU: act(g) = g * (1/(1+exp(-g))); the gated GELU uses the tanh form
0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from .base import FeedForward, TensorSpec, register_feed_forward
from .linear import Linear


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """params: width, inter.  tensors: gate_proj/up_proj/down_proj .weight (or the three names in ``names``)."""

    graph_safe = True
    launches_through_ops = True
    act = ops.ACT_SILU
    default_names = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.width, self.inter = int(params["width"]), int(params["inter"])
        self.names = tuple(params.get("names", self.default_names))
        if len(self.names) != 3:
            raise ValueError("a gated feed-forward has three tensors: gate, up, down")
        self.gate_up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {
            self.names[0]: TensorSpec((self.inter, self.width)),
            self.names[1]: TensorSpec((self.inter, self.width)),
            self.names[2]: TensorSpec((self.width, self.inter)),
        }

    def bind(self, tensors) -> None:
        g, u = tensors[self.names[0]], tensors[self.names[1]]
        if g.dtype != u.dtype:
            raise ValueError("gate and up projections must be stored in one dtype to be stacked")
        self.gate_up = Linear(torch.cat([g, u], dim=0), self.rt)
        self.down = Linear(tensors[self.names[2]], self.rt)

    def weight_bytes(self) -> int:
        return self.gate_up.nbytes() + self.down.nbytes()

    def forward_with_norm(self, ctx, x, norm, residual) -> bool:
        """Decode steps of few rows: norm, the stacked product and SwiGLU are one kernel."""
        from .norm import RMSNorm
        rt, ws = self.rt, ctx.ws
        if not (rt.bf16 and isinstance(norm, RMSNorm) and self.gate_up.mfma and self.down.mfma
                and ops.can_fuse_norm(ctx.rows, self.gate_up.weight, x, columns=32, stacked=2)):
            return False
        act = ws.buffer("mlp_h", self.inter, torch.bfloat16)
        ops.norm_gemm_bf16(x, norm.weight, norm.eps, self.gate_up.weight, act, ctx.rows, ops.EPI_SWIGLU_BF16)
        self.down.add_into(ws, act, residual, ctx.rows)
        return True

    def forward(self, ctx, h, residual) -> None:
        rt, ws, rows = self.rt, ctx.ws, ctx.rows
        if self.gate_up.mfma:
            act = ws.buffer("mlp_h", self.inter, torch.bfloat16)
            ops.gemm_bf16(h, self.gate_up.weight, act, rows, ops.EPI_SWIGLU_BF16)   # SwiGLU in the epilogue
        else:
            gu = ws.buffer("gate_up", 2 * self.inter, torch.float32)
            self.gate_up.store(ws, h, gu, rows)
            act32 = ws.buffer("mlp_h32", self.inter, torch.float32)
            ops.swiglu_f32(gu, act32, rows)
            if rt.bf16:
                # bfloat16 mode rounds the activation here whatever dtype the weights are stored in, so that
                # the mode has one set of rounding points (a 32-bit down projection widens it again)
                act = ws.buffer("mlp_h", self.inter, torch.bfloat16)
                ops.convert(act32, act, rows)
            else:
                act = act32
        self.down.add_into(ws, act, residual, rows)


@register_feed_forward("geglu")
class GeGLU(SwiGLU):
    """The same arrangement with the tanh form of GELU on the gate.  The stacked product leaves 32-bit sums; the
    activation and the product with ``up`` are one 32-bit kernel behind it, which rounds once for the down projection."""

    act = ops.ACT_GELU_TANH
    default_names = ("gate", "up", "down")

    def forward_with_norm(self, ctx, x, norm, residual) -> bool:
        """Decode steps of few rows: the norm rides in the stacked product (the bits of norm, then product)."""
        from .norm import RMSNorm
        ws, rows = ctx.ws, ctx.rows
        if not (self.rt.bf16 and type(norm) is RMSNorm and self.gate_up.mfma and ops.can_fuse_norm(rows, self.gate_up.weight, x)):
            return False
        gu = ws.buffer("gate_up", 2 * self.inter, torch.float32)
        ops.norm_gemm_bf16(x, norm.weight, norm.eps, self.gate_up.weight, gu, rows, ops.EPI_F32)
        self._gate_and_down(ctx, gu, residual)
        return True

    def _gate_and_down(self, ctx, gu, residual) -> None:
        act = ctx.ws.buffer("mlp_h", self.inter, self.rt.act_dtype)
        ops.glu(gu, act, ctx.rows, self.act, **self._act_params())
        self.down.add_into(ctx.ws, act, residual, ctx.rows)

    def _act_params(self) -> dict:
        return {}

    def forward(self, ctx, h, residual) -> None:
        gu = ctx.ws.buffer("gate_up", 2 * self.inter, torch.float32)
        self.gate_up.store(ctx.ws, h, gu, ctx.rows)
        self._gate_and_down(ctx, gu, residual)


@register_feed_forward("clamped_glu")
class ClampedGLU(GeGLU):
    """The same arrangement with a clamped gate and a shifted up branch:

        g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit), y = g sigmoid(alpha g) (u + 1), out = W_down y

    params: width, inter, limit, alpha (1.702), names.  Prompt portions of more than 64 rows compute the activation in the
    stacked product's epilogue (bfloat16 mode, weights the matrix cores take); otherwise it is one 32-bit kernel behind the
    product.  Both are the same sequence of operations on the same 32-bit sums, so a row's bits do not depend on the route."""

    act = ops.ACT_CLAMPED_SWISH

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.limit, self.alpha = float(params["limit"]), float(params.get("alpha", 1.702))
        if not self.limit > 0:
            raise ValueError("clamped_glu: the limit must be positive")

    def _act_params(self) -> dict:
        return {"limit": self.limit, "alpha": self.alpha}

    def forward(self, ctx, h, residual) -> None:
        if self.rt.bf16 and self.gate_up.mfma and self.gate_up.bias is None and ctx.rows >= ops.CLAMPED_GLU_MIN_ROWS:
            act = ctx.ws.buffer("mlp_h", self.inter, torch.bfloat16)
            ops.gemm_clamped_glu_bf16(h, self.gate_up.weight, act, ctx.rows, self.limit, self.alpha)
            self.down.add_into(ctx.ws, act, residual, ctx.rows)
        else:
            super().forward(ctx, h, residual)
