"""Token embedding and the language-model head (src/model.cpp:274, :308-321)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from .base import Embedding, Head, StateSpec, TensorSpec, register_embedding, register_head
from .linear import Linear


@register_embedding("embedding")
class TokenEmbedding(Embedding):
    """params: vocab, width; optional ``norm`` = {tensor, eps}: the gathered row is divided by its root mean square and
    multiplied by that weight vector before it becomes the stream.  tensor: weight [vocab, width], gathered as 32-bit rows."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.vocab, self.width = int(params["vocab"]), int(params["width"])
        self.tensor = str(params.get("tensor", "weight"))      # the table's name behind the prefix
        self.weight: Optional[torch.Tensor] = None
        self.norm = dict(params["norm"]) if params.get("norm") else None
        self.norm_weight: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        out = {self.tensor: TensorSpec((self.vocab, self.width), "embedding")}
        if self.norm is not None:
            out[str(self.norm["tensor"])] = TensorSpec((self.width,), "norm")
        return out

    def bind(self, tensors) -> None:
        self.weight = tensors[self.tensor].to(self.rt.device).contiguous()
        if self.norm is not None:
            self.norm_weight = tensors[str(self.norm["tensor"])].to(self.rt.device).float().contiguous()

    def weight_bytes(self) -> int:
        return 0      # a step reads one row per token, not the table

    def forward(self, ctx) -> torch.Tensor:
        x = ctx.ws.buffer("residual", self.width, torch.float32)
        # (a step launched ahead of its tokens names them by the step before: ``ctx.token_feedback``)
        if self.norm is None:
            ops.embed(ctx.tokens[:ctx.rows], self.weight, x, getattr(ctx, "token_feedback", None))
            return x
        rows = ctx.ws.buffer("embedded_rows", self.width, torch.float32)
        ops.embed(ctx.tokens[:ctx.rows], self.weight, rows, getattr(ctx, "token_feedback", None))
        ops.rmsnorm(rows, self.norm_weight, x, ctx.rows, float(self.norm["eps"]))
        return x


@register_embedding("embedding_sum")
class SummedEmbedding(TokenEmbedding):
    """The token's row times a scale, plus (each optional) a row of a table of token pairs and a learned row per position:

        x = table[token] * scale + pairs[(token before * mul_prev + token * mul_cur) mod buckets] + positions[p]

    A request's first token takes the pair table's last row (number ``buckets``).  The token before a step's first token
    of a request is per-request state (one word), so that a prompt may be cut anywhere.  All 32-bit.
    params: vocab, width, tensor, scale (1); ``pairs``: None or {tensor, buckets, mul_prev, mul_cur}; ``positions``: None or
    {tensor, count}."""

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.scale = float(params.get("scale", 1.0))
        self.pairs = dict(params["pairs"]) if params.get("pairs") else None
        self.positions = dict(params["positions"]) if params.get("positions") else None
        if self.pairs is not None:
            b, mp, mc = int(self.pairs["buckets"]), int(self.pairs["mul_prev"]), int(self.pairs["mul_cur"])
            if b < 1 or mp < 0 or mc < 0:
                raise ValueError("embedding_sum: the pair table needs at least one bucket and multipliers that are not negative")
            self.pair_hash = (b, mp, mc)
        self.pair_table = self.pos_table = None

    def tensors(self) -> Dict[str, TensorSpec]:
        out = super().tensors()
        if self.pairs is not None:
            out[str(self.pairs["tensor"])] = TensorSpec((self.pair_hash[0] + 1, self.width), "embedding")
        if self.positions is not None:
            out[str(self.positions["tensor"])] = TensorSpec((int(self.positions["count"]), self.width), "embedding")
        return out

    def bind(self, tensors) -> None:
        super().bind(tensors)
        put = lambda t: t.to(self.rt.device).to(self.weight.dtype).contiguous()     # (one dtype for the kernel; the same values)
        if self.pairs is not None:
            self.pair_table = put(tensors[str(self.pairs["tensor"])])
        if self.positions is not None:
            self.pos_table = put(tensors[str(self.positions["tensor"])])
        stored = {t.dtype for t in tensors.values()}
        if len(stored) != 1:
            raise ValueError("embedding_sum: the tables must be stored in one dtype")

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((1,), "int32") if self.pairs is not None else None

    def forward(self, ctx) -> torch.Tensor:
        x = ctx.ws.buffer("residual", self.width, torch.float32)
        state = getattr(ctx, "embedding_state", None)
        if self.pairs is not None and state is None:
            raise ValueError("embedding_sum: the step's context carries no state for the embedding (the token before)")
        ops.embed_sum(ctx.tokens[:ctx.rows], ctx.positions, self.weight, self.scale, x,
                      pair_table=self.pair_table, pair_hash=self.pair_hash if self.pairs is not None else (0, 0, 0),
                      pos_table=self.pos_table, row_seq=ctx.row_seq, seq_rows=ctx.seq_rows, slots=ctx.slots, state=state,
                      feedback=getattr(ctx, "token_feedback", None))
        return x


@register_head("lm_head")
class LMHead(Head):
    """params: vocab, width, tied; optional ``scale``: the logits are multiplied by it (one 32-bit product each).
    tensor: weight [vocab, width] unless tied to the embedding (src/model.cpp:170-171).  Only the wanted rows are normed
    and projected."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.vocab, self.width, self.tied = int(params["vocab"]), int(params["width"]), bool(params["tied"])
        self.tensor = str(params.get("tensor", "weight"))
        self.scale = float(params.get("scale", 1.0))
        self.linear: Optional[Linear] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {} if self.tied else {self.tensor: TensorSpec((self.vocab, self.width), "linear")}

    def bind(self, tensors, embedding=None) -> None:
        if self.tied:
            table = getattr(embedding, "weight", None)
            if table is None or tuple(table.shape) != (self.vocab, self.width):
                raise ValueError("a tied head needs an embedding part with a table [vocab, width]")
            self.linear = Linear(table, self.rt)     # the same device tensor, not a copy
        else:
            self.linear = Linear(tensors[self.tensor], self.rt)

    def weight_bytes(self) -> int:
        return self.linear.nbytes()

    def forward(self, ctx, x: torch.Tensor, norm, count: int) -> torch.Tensor:
        """Final norm and projection of ``count`` rows; few rows: both are one kernel (the same bits)."""
        from .norm import RMSNorm
        ws = ctx.ws
        logits = ws.buffer("logits", self.vocab, torch.float32, rows=ws.max_logit_rows)
        if (self.rt.bf16 and isinstance(norm, RMSNorm) and self.linear.mfma
                and ops.can_fuse_norm(count, self.linear.weight, x)):
            ops.norm_gemm_bf16(x, norm.weight, norm.eps, self.linear.weight, logits, count, ops.EPI_F32)
        else:
            normed = norm.forward(ctx, x, out_name="final_normed", rows=count)
            self.linear.store(ws, normed, logits, count)
        if self.scale != 1.0:
            ops.scale_rows(logits, count, self.scale)
        return logits


@register_head("lm_head_softcap")
class SoftCappedLMHead(LMHead):
    """``lm_head`` whose logits are squashed: logits <- cap * tanh(logits / cap), 32-bit, in place.  params as LMHead, plus ``cap``."""

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.cap = float(params["cap"])
        if not self.cap > 0:
            raise ValueError("lm_head_softcap: the cap must be positive")

    def forward(self, ctx, x: torch.Tensor, norm, count: int) -> torch.Tensor:
        logits = super().forward(ctx, x, norm, count)
        ops.softcap(logits, count, self.cap)
        return logits
