"""A feed-forward of routed experts: every row goes through the ``top`` experts its router scores pick, and their
outputs are added with the scores as weights.

    s       = softmax(W_router h)                              over all experts, 32-bit (``score`` "sigmoid": the sigmoid of each logit)
    c       = s, or s + correction                             a learned number per expert that enters the choice only
    allowed = the experts of the `keep` best of `groups` equal groups of neighbours (a group's score: its best c, or
              with ``group_best`` n the sum of its n best)
    chosen  = the `top` allowed experts with the largest c; weights = their s, as they are
    expert  : g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit), W_down (g sigmoid(alpha g) (u + 1))
              or, with limit None, the plain gated form W_down (g sigmoid(alpha g) u), g = W_gate h, u = W_up h

``weight_scale`` multiplies the chosen scores.  ``shared`` = {ff}: one more expert of the plain gated form (tensors
shared.gate, shared.up, shared.down) that every row goes through, its output multiplied by sigmoid(w_sg . h), one number
a row (tensor shared.sg [1, width]); the gate's product rides under the router's, 32-bit like it.  ``shared`` =
{ff, "gated": False}: the shared expert's output is added as it is (no tensor shared.sg).

Routing happens on the device and the experts' products run over a plan built there, so a step never waits for the
host and a captured decode step stays valid.  What a row gets from an expert depends on the row and the expert
alone, whatever else is in the batch.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from .base import FeedForward, TensorSpec, register_feed_forward
from .linear import Linear


@register_feed_forward("moe")
class RoutedExperts(FeedForward):
    """params: width, experts, top, groups (1), keep (groups), ff, limit (None: the plain form), alpha (1.702; 1 makes the
    plain form SiLU), weight_scale (1), shared (None or {ff, gated (True)}), score ("softmax" or "sigmoid"), correction
    (False; True: a tensor ``correction`` [experts] joins the scores for the choice), group_best (1).
    tensors: router [experts, width]; e<j>.gate, e<j>.up [ff, width]; e<j>.down [width, ff]; with ``shared``:
    shared.gate, shared.up [ff_s, width], shared.down [width, ff_s], shared.sg [1, width] if gated; correction [experts]."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        p = params
        self.width, self.experts, self.top, self.ff = int(p["width"]), int(p["experts"]), int(p["top"]), int(p["ff"])
        self.groups = int(p.get("groups", 1))
        self.keep = int(p.get("keep", self.groups))
        self.limit = 0.0 if p.get("limit") is None else float(p["limit"])       # (0 tells the kernels: the plain form)
        self.alpha = float(p.get("alpha", 1.702))
        self.weight_scale = float(p.get("weight_scale", 1.0))
        self.shared_ff = int(p["shared"]["ff"]) if p.get("shared") else 0
        self.shared_gated = bool(p["shared"].get("gated", True)) if p.get("shared") else False
        if p.get("score", "softmax") not in ("softmax", "sigmoid"):
            raise ValueError(f"moe: scores are 'softmax' or 'sigmoid', not {p.get('score')!r}")
        self.score = ops.SCORE_SIGMOID if p.get("score") == "sigmoid" else ops.SCORE_SOFTMAX
        self.has_correction = bool(p.get("correction", False))
        self.group_best = int(p.get("group_best", 1))
        if not 1 <= self.group_best <= 4:
            raise ValueError("moe: a group's score sums one to four of its best")
        self.correction: Optional[torch.Tensor] = None
        if p.get("limit") is not None and not self.limit > 0:
            raise ValueError("moe: the experts' limit must be positive (None: no limit)")
        if self.experts % self.groups or not 1 <= self.keep <= self.groups:
            raise ValueError(f"moe: {self.experts} experts in {self.groups} groups of which {self.keep} are kept")
        if not 1 <= self.top <= self.keep * (self.experts // self.groups):
            raise ValueError(f"moe: {self.top} experts a row out of {self.keep} groups of {self.experts // self.groups}")
        self.router: Optional[Linear] = None
        self.gate_up = self.down = None
        self.shared_gate_up: Optional[Linear] = None       # (None with a shared expert: its two branches ride under the router)
        self.shared_at = 0                                 # the column of the router's product where they begin
        self.shared_down: Optional[Linear] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        out = {}
        for j in range(self.experts):
            out[f"e{j}.gate"] = TensorSpec((self.ff, self.width))
            out[f"e{j}.up"] = TensorSpec((self.ff, self.width))
            out[f"e{j}.down"] = TensorSpec((self.width, self.ff))
        out["router"] = TensorSpec((self.experts, self.width), "router")
        if self.shared_ff:
            out["shared.gate"] = TensorSpec((self.shared_ff, self.width))
            out["shared.up"] = TensorSpec((self.shared_ff, self.width))
            out["shared.down"] = TensorSpec((self.width, self.shared_ff))
            if self.shared_gated:
                out["shared.sg"] = TensorSpec((1, self.width), "router")
        if self.has_correction:
            out["correction"] = TensorSpec((self.experts,), "small_bias")
        return out

    def bind(self, tensors) -> None:
        dev = self.rt.device
        # the router's sums are 32-bit in either mode; in bfloat16 mode the rows arrive rounded and the weights are stored
        # so, their products are exact in 32 bits and the matrix cores add them up in 32 bits
        if self.has_correction:
            self.correction = tensors["correction"].to(dev).float().contiguous()
        if self.shared_ff:
            if tensors["shared.gate"].dtype != tensors["shared.up"].dtype or (
                    self.shared_gated and tensors["shared.sg"].dtype != tensors["router"].dtype):
                raise ValueError("the router and the shared expert's gate (and its two branches) must be stored in one dtype to be stacked")
            under = [tensors["router"]] + ([tensors["shared.sg"]] if self.shared_gated else [])
            if tensors["shared.gate"].dtype == tensors["router"].dtype:
                # one product gives the experts' logits, the shared expert's gate and its two branches: all read the same
                # rows and all leave 32-bit sums (a product's column does not depend on the columns beside it)
                self.router = Linear(torch.cat(under + [tensors["shared.gate"], tensors["shared.up"]], dim=0), self.rt)
                self.shared_at = sum(t.shape[0] for t in under)
            else:
                self.router = Linear(torch.cat(under, dim=0), self.rt)
                self.shared_gate_up = Linear(torch.cat([tensors["shared.gate"], tensors["shared.up"]], dim=0), self.rt)
            self.shared_down = Linear(tensors["shared.down"], self.rt)
        else:
            self.router = Linear(tensors["router"], self.rt)
        kinds = {tensors[f"e{j}.{n}"].dtype for j in range(self.experts) for n in ("gate", "up", "down")}
        if len(kinds) != 1:
            raise ValueError("the experts of one feed-forward must be stored in one dtype to be stacked")
        self.gate_up = torch.stack([torch.cat([tensors[f"e{j}.gate"], tensors[f"e{j}.up"]], dim=0) for j in range(self.experts)]).to(dev).contiguous()
        self.down = torch.stack([tensors[f"e{j}.down"] for j in range(self.experts)]).to(dev).contiguous()
        self.mfma = bool(self.rt.bf16 and self.gate_up.dtype == torch.bfloat16 and self.width % 8 == 0 and self.ff % 8 == 0)

    def weight_bytes(self) -> int:
        """Bytes a decode step of one row reads: the router and the chosen experts."""
        per = (self.gate_up.numel() + self.down.numel()) // self.experts * self.gate_up.element_size()
        return self.router.nbytes() + self.top * per + self._shared_bytes()

    def _shared_bytes(self) -> int:
        if not self.shared_ff:
            return 0
        return (0 if self.shared_gate_up is None else self.shared_gate_up.nbytes()) + self.shared_down.nbytes()

    def weight_bytes_rows(self, rows: int) -> int:
        """Bytes a decode step of ``rows`` rows reads: the router and the experts the rows touch, on average, if every
        expert is as likely as any other: experts * (1 - (1 - top/experts)^rows)."""
        per = (self.gate_up.numel() + self.down.numel()) // self.experts * self.gate_up.element_size()
        touched = self.experts * (1.0 - (1.0 - self.top / self.experts) ** max(int(rows), 1))
        return self.router.nbytes() + int(touched * per) + self._shared_bytes()

    def _run(self, ctx, h, target, add: bool, norm=None, rounded=None) -> None:
        rt, ws, rows = self.rt, ctx.ws, ctx.rows
        slots = rows * self.top
        most = ws.max_rows * self.top
        logits = ws.buffer("moe_logits", self.router.out_features, torch.float32)
        self.router.store(ws, h, logits, rows)
        ids = ws.buffer("moe_ids", self.top, torch.int32)
        wts = ws.buffer("moe_wts", self.top, torch.float32)
        sorted_slots = ws.buffer("moe_sorted", most, torch.int32, rows=1)
        place = ws.buffer("moe_place", most, torch.int32, rows=1)
        # (room for the plan of any step: tiles hold 16 slots or more, and every expert may end with a partly filled one)
        tiles = ws.buffer("moe_tiles", 4 * (most // 16 + self.experts), torch.int32, rows=1)
        meta = ws.buffer("moe_meta", 4, torch.int32, rows=1)
        ops.moe_route_plan(logits, rows, self.top, self.groups, self.keep, ids, wts, sorted_slots, place, tiles, meta,
                           weight_scale=self.weight_scale, experts=self.experts, score=self.score, correction=self.correction,
                           group_best=self.group_best)
        if self.mfma:
            x, act_dtype = h, torch.bfloat16
        else:
            x, act_dtype = h, torch.float32
            if h.dtype != torch.float32:
                x = ws.buffer("moe_x32", self.width, torch.float32)
                ops.convert(h, x, rows)
        act = ws.buffer("moe_act", self.ff, act_dtype, rows=most)
        ops.moe_experts(x, self.gate_up, act, sorted_slots, tiles, meta, slots, self.top, True, self.limit, self.alpha,
                        round_out=rt.bf16 and not self.mfma)
        y = ws.buffer("moe_y", self.width, torch.float32, rows=most)
        ops.moe_experts(act, self.down, y, sorted_slots, tiles, meta, slots, self.top, False)
        if norm is not None:
            # the rows' weighted sums are formed by the kernel that norms them and adds them into the stream
            ops.norm_add(y, norm.weight, target, rows, norm.eps, rounded, combine=(place, wts, self.top), scale=norm.scale)
        else:
            ops.moe_combine(y, place, wts, self.top, target, rows, add)
        if self.shared_ff:
            # the shared expert: its activation takes the row's gate with it, so that its down projection adds straight
            # into the target
            if self.shared_gate_up is None:
                gu = logits[:, self.shared_at:self.shared_at + 2 * self.shared_ff]
            else:
                gu = ws.buffer("moe_shared_gu", 2 * self.shared_ff, torch.float32)
                self.shared_gate_up.store(ws, h, gu, rows)
            sact = ws.buffer("moe_shared_act", self.shared_ff, rt.act_dtype)
            ops.glu(gu, sact, rows, ops.ACT_SILU, row_gate=logits[:, self.experts:self.experts + 1] if self.shared_gated else None)
            self.shared_down.add_into(ws, sact, target, rows)

    def forward(self, ctx, h, residual) -> None:
        self._run(ctx, h, residual, True)

    def forward_out(self, ctx, h, out) -> None:
        self._run(ctx, h, out, False)

    def forward_add_normed(self, ctx, h, norm, x, rounded=None) -> bool:
        from .norm import RMSNorm
        # (few rows: a launch that sums the choices over many workgroups and the norm's own launch are faster than one
        # workgroup a row doing both; the bits are the same either way)
        if type(norm) is not RMSNorm or ctx.rows <= 16 or self.shared_ff:
            return False
        self._run(ctx, h, x, True, norm=norm, rounded=rounded)
        return True
