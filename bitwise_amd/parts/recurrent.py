"""Mixers with a matrix memory per head instead of a cache: S <- decay * S + k v^T, o = S^T q.

Four kinds share the arrangement (one stacked projection of the mixer's input, the recurrence over each request's
rows in order from and to its state slot, a per-head RMS norm of the read-out with an output gate, the output
projection added into the residual stream) and differ in the decay:

* ``gla``: gated linear attention, a decay per key channel, alpha = sigmoid(z)^(1/tau) with z a low-rank
  projection of the input plus a bias; the read-out norm has one weight vector for all heads and the gate is SiLU.
* ``mlstm``: the matrix memory of the xLSTM, scalar input and forget gates per head in the log domain, capped by
  cap * tanh(. / cap), with a normaliser n and a stabilising maximum m (a new request's m is 0, like the rest of its
  state); the read-out is divided by max(|n.q|, exp(-m)) + 1e-6, the norm weight spans all heads and the gate is a sigmoid.
* ``wkv``: time mixing in the manner of RWKV: every projection reads its own mix of the token's and the previous token's
  input (the norm in front of the mixer delivers the mixes side by side), the decay per key channel is
  exp(-exp(W2 tanh(W1 x) + w0)), and the read-out comes before the update, with the token's own k v^T weighted by a
  learned bonus: o = (S + diag(u) k v^T)^T r, then S <- diag(decay) S + k v^T; SiLU gate, norm weight over all heads.
* ``retention``: one constant decay per head, queries and keys rotated by position (halves layout) and the keys scaled by
  dim^(-1/2) behind the rotation; the read-out norm has no weight and the gate is SiLU.

The state, the gates and everything between the projections and the read-out are 32-bit in both modes; the
projections' sums arrive as 32-bit values and are not rounded on the way.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from ..csrc import ops
from .base import Mixer, POSITION_ENCODINGS, StateSpec, TensorSpec, lookup, register_mixer
from .linear import Linear


SCAN_CHUNK = 32          # rows of a chunk of a long portion
SCAN_MIN_ROWS = 96       # portions from this many rows on run in three passes over chunks (shorter ones: one wave each),
                         # where the engine allows logits to depend on the cut in their last bits (Workspace.exact_cuts False)


def _scan_plan(ctx):
    """Which requests of the step bring long portions, cut into chunks: (seq_rows for the others, their count, chunks,
    number of chunks, spans, number of spans), or None if every portion is short (a step of single tokens always is).  One
    plan a step, shared by its layers."""
    if getattr(ctx, "one_row_per_request", False) or getattr(ctx.ws, "exact_cuts", True):
        return None

    def make():
        long = [i for i, s in enumerate(ctx.segments) if len(s.tokens) >= SCAN_MIN_ROWS]
        if not long:
            return None
        short_rows = np.asarray([(ctx.seq_start[i], 0 if i in long else len(s.tokens)) for i, s in enumerate(ctx.segments)],
                                np.int32).reshape(-1)
        chunks, spans = [], []
        for i in long:
            n, r0 = len(ctx.segments[i].tokens), ctx.seq_start[i]
            first_chunk = len(chunks)
            for off in range(0, n, SCAN_CHUNK):
                chunks.append((r0 + off, min(SCAN_CHUNK, n - off), i, 1 if off + SCAN_CHUNK >= n else 0))
            spans.append((i, first_chunk, len(chunks) - first_chunk))
        flat = np.concatenate([short_rows, np.asarray(chunks, np.int32).reshape(-1), np.asarray(spans, np.int32).reshape(-1)])
        dev = torch.from_numpy(flat).to(ctx.device)
        a, b = short_rows.size, short_rows.size + 4 * len(chunks)
        any_short = len(long) < len(ctx.segments)
        return dev[:a], (ctx.nseq if any_short else 0), dev[a:b], len(chunks), dev[b:], len(spans)

    return ctx.memo(("recurrence_scan_plan",), make)


class _MatrixMemoryMixer(Mixer):
    """params: width, heads, dim (key channels a head), vdim (value channels a head), eps (of the read-out norm);
    optional ``names``: the tensors' names behind the prefix."""

    graph_safe = True
    launches_through_ops = True
    mode = -1
    gate_kind = ops.GATE_SIGMOID
    per_head_norm_weight = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        p = params
        self.width, self.heads, self.dim, self.vdim = int(p["width"]), int(p["heads"]), int(p["dim"]), int(p["vdim"])
        self.eps = float(p["eps"])
        if self.dim > ops.RECUR_MAX_DIM:
            raise ValueError(f"{type(self).__name__}: {self.dim} key channels a head; the kernel keeps up to {ops.RECUR_MAX_DIM}")
        self.qscale = float(self.dim) ** -0.5
        self.proj: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.norm_weight: Optional[torch.Tensor] = None
        self.offsets: Dict[str, int] = {}
        self.proj_width = 0

    # -- sizes of the stacked projections, in order
    def _stack_sizes(self) -> List[Tuple[str, int]]:
        raise NotImplementedError

    def _norm_weight_size(self) -> int:
        return self.heads * self.vdim if self.per_head_norm_weight else self.vdim

    def tensors(self) -> Dict[str, TensorSpec]:
        out = {name: TensorSpec((n, self.width)) for name, n in self._stack_sizes()}
        out["o"] = TensorSpec((self.width, self.heads * self.vdim))
        out["norm"] = TensorSpec((self._norm_weight_size(),), "norm")
        return out

    def _bind_common(self, tensors) -> None:
        parts = [tensors[name] for name, _ in self._stack_sizes()]
        if len({t.dtype for t in parts}) != 1:
            raise ValueError("the projections of one mixer must be stored in one dtype to be stacked")
        off = 0
        for name, n in self._stack_sizes():
            self.offsets[name] = off
            off += n
        self.proj_width = off
        self.proj = Linear(torch.cat(parts, dim=0), self.rt)
        self.o = Linear(tensors["o"], self.rt)
        self.norm_weight = tensors["norm"].to(self.rt.device).float().contiguous()

    def state_spec(self) -> StateSpec:
        n = self.heads * self.dim * self.vdim
        if self.mode == ops.RECUR_SCALAR_GATES:
            n += self.heads * self.dim + self.heads
        return StateSpec((n,), "float32")

    def input_projection(self):
        return self.proj

    def adopt_input_projection(self, weight) -> None:
        self.proj = Linear(weight, self.rt)

    def _project(self, ctx, h) -> torch.Tensor:
        """The stacked projection of the rows as 32-bit sums."""
        y = ctx.ws.buffer("recur_proj", self.proj_width, torch.float32)
        self.proj.store(ctx.ws, h, y, ctx.rows)
        return y

    def _recur(self, ctx, call, y, gate, gate_off, gate2_off, bias, bias2, param, raw, kscale: float = 1.0, at=None) -> None:
        """``at``: where q (or r), k and v lie in a row of ``y``, if not at the stacked projection's own offsets."""
        at = self.offsets if at is None else at
        plan = _scan_plan(ctx)
        seq_rows, nseq, scan = ctx.seq_rows, ctx.nseq, None
        if plan is not None:
            seq_rows, nseq, chunks, nchunks, spans, nspans = plan
            rec = self.heads * (self.dim * self.vdim + self.dim + 2)
            most = ctx.ws.max_rows // SCAN_CHUNK + ctx.ws.max_rows // SCAN_MIN_ROWS + 1     # chunks a step can bring
            local = ctx.ws.buffer("recur_scan_local", most * rec, torch.float32, rows=1)
            start = ctx.ws.buffer("recur_scan_start", most * rec, torch.float32, rows=1)
            scan = (chunks, nchunks, spans, nspans, local, start)
        ops.linear_recurrence(self.mode, y, at["r"] if "q" not in at else at["q"], at["k"], at["v"], gate, gate_off, gate2_off,
                              bias, bias2, param, self.qscale, call.state, raw, seq_rows, ctx.slots, ctx.positions, nseq,
                              self.heads, self.dim, self.vdim, scan=scan, kscale=kscale)

    def _finish(self, ctx, y, raw, target, add: bool = True, g_off: Optional[int] = None) -> None:
        act = ctx.ws.buffer("recur_gated", self.heads * self.vdim, self.rt.act_dtype)
        ops.head_norm_gate(raw, self.norm_weight, self.per_head_norm_weight, y, self.offsets["g"] if g_off is None else g_off, self.gate_kind, act,
                           ctx.positions, ctx.rows, self.heads, self.vdim, self.eps)
        if add:
            self.o.add_into(ctx.ws, act, target, ctx.rows)
        else:
            self.o.store(ctx.ws, act, target, ctx.rows)


@register_mixer("gla")
class GatedLinearAttention(_MatrixMemoryMixer):
    """params as the base, plus tau and rank (the inner size of the decay's low-rank projection).
    tensors: q, k [heads*dim, width]; v, g [heads*vdim, width]; a1 [rank, width]; a2 [heads*dim, rank]; a2.b [heads*dim];
    norm [vdim]; o [width, heads*vdim]."""

    mode = ops.RECUR_DECAY_PER_CHANNEL
    gate_kind = ops.GATE_SILU
    per_head_norm_weight = False

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.tau, self.rank = float(params["tau"]), int(params["rank"])
        if self.tau <= 0:
            raise ValueError("gla: tau must be positive")
        self.a2: Optional[Linear] = None
        self.a2_bias: Optional[torch.Tensor] = None

    def _stack_sizes(self):
        hd, hv = self.heads * self.dim, self.heads * self.vdim
        return [("q", hd), ("k", hd), ("v", hv), ("g", hv), ("a1", self.rank)]

    def tensors(self):
        out = super().tensors()
        out["a2"] = TensorSpec((self.heads * self.dim, self.rank))
        out["a2.b"] = TensorSpec((self.heads * self.dim,), "bias")
        return out

    def bind(self, tensors) -> None:
        self._bind_common(tensors)
        # the inner size is tiny and its input stays 32-bit: the 32-bit kernels in either mode
        self.a2 = Linear(tensors["a2"], self.rt, matrix_cores=False)
        self.a2_bias = tensors["a2.b"].to(self.rt.device).float().contiguous()

    def weight_bytes(self) -> int:
        return self.proj.nbytes() + self.o.nbytes() + self.a2.nbytes() + 4 * (self.a2_bias.numel() + self.norm_weight.numel())

    def forward(self, ctx, call, h, residual) -> None:
        ws, rows = ctx.ws, ctx.rows
        y = self._project(ctx, h)
        low = y[:, self.offsets["a1"]:self.offsets["a1"] + self.rank]      # (a view: the product reads it in place)
        z = ws.buffer("gla_decay_logits", self.heads * self.dim, torch.float32)
        self.a2.store(ws, low, z, rows)
        raw = ws.buffer("recur_out", self.heads * self.vdim, torch.float32)
        self._recur(ctx, call, y, z, 0, 0, self.a2_bias, None, 1.0 / self.tau, raw)
        self._finish(ctx, y, raw, residual)


@register_mixer("mlstm")
class MatrixLSTM(_MatrixMemoryMixer):
    """params as the base, plus gate_cap.  tensors: q, k [heads*dim, width]; v, g [heads*vdim, width]; i, f [heads, width];
    i.b, f.b [heads]; norm [heads*vdim]; o [width, heads*vdim]."""

    mode = ops.RECUR_SCALAR_GATES
    gate_kind = ops.GATE_SIGMOID
    per_head_norm_weight = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.cap = float(params["gate_cap"])
        if self.cap <= 0:
            raise ValueError("mlstm: gate_cap must be positive")
        self.i_bias: Optional[torch.Tensor] = None
        self.f_bias: Optional[torch.Tensor] = None

    def _stack_sizes(self):
        hd, hv = self.heads * self.dim, self.heads * self.vdim
        return [("q", hd), ("k", hd), ("v", hv), ("g", hv), ("i", self.heads), ("f", self.heads)]

    def tensors(self):
        out = super().tensors()
        out["i.b"] = TensorSpec((self.heads,), "bias")
        out["f.b"] = TensorSpec((self.heads,), "bias")
        return out

    def bind(self, tensors) -> None:
        self._bind_common(tensors)
        self.i_bias = tensors["i.b"].to(self.rt.device).float().contiguous()
        self.f_bias = tensors["f.b"].to(self.rt.device).float().contiguous()

    def weight_bytes(self) -> int:
        return self.proj.nbytes() + self.o.nbytes() + 4 * (2 * self.heads + self.norm_weight.numel())

    def forward(self, ctx, call, h, residual) -> None:
        y = self._project(ctx, h)
        raw = ctx.ws.buffer("recur_out", self.heads * self.vdim, torch.float32)
        self._recur(ctx, call, y, y, self.offsets["i"], self.offsets["f"], self.i_bias, self.f_bias, self.cap, raw)
        self._finish(ctx, y, raw, residual)


@register_mixer("wkv")
class TimeMixWKV(_MatrixMemoryMixer):
    """params: width, heads, dim (key and value channels a head), eps, rank (the inner size of the decay's projection),
    inputs (the names of the mixes the norm in front delivers side by side, in its order; this mixer reads "r", "k", "v",
    "g" and "w" among them).
    tensors: r, k, v, g [heads*dim, width]; w1 [rank, width]; w2 [heads*dim, rank]; w0 [heads*dim]; u [heads, dim];
    norm [heads*dim]; o [width, heads*dim].  The mixer's input is [rows, len(inputs) * width]."""

    mode = ops.RECUR_BONUS_DECAY
    gate_kind = ops.GATE_SILU
    per_head_norm_weight = True
    READS = ("r", "k", "v", "g", "w")

    def __init__(self, params, runtime):
        params = dict(params, vdim=int(params["dim"]))
        super().__init__(params, runtime)
        self.qscale = 1.0                     # (the receptance enters the read-out as it is)
        self.rank = int(params["rank"])
        self.inputs = [str(n) for n in params.get("inputs", self.READS)]
        missing = [n for n in self.READS if n not in self.inputs]
        if missing or self.rank < 1:
            raise ValueError(f"wkv: the norm in front must deliver the mixes {missing}; the decay's inner size must be positive")
        self.lin: Dict[str, Linear] = {}
        self.w2: Optional[Linear] = None
        self.w0 = self.bonus = None

    def _stack_sizes(self):
        hd = self.heads * self.dim
        return [("r", hd), ("k", hd), ("v", hd), ("g", hd), ("w1", self.rank)]

    def tensors(self):
        out = super().tensors()
        hd = self.heads * self.dim
        out["w2"] = TensorSpec((hd, self.rank))
        out["w0"] = TensorSpec((hd,), "small_bias")
        out["u"] = TensorSpec((self.heads, self.dim), "small_bias")
        return out

    FEW_ROWS = 12          # steps of up to this many rows run the five projections as one product (below)

    def bind(self, tensors) -> None:
        dev = self.rt.device
        names = [name for name, _ in self._stack_sizes()]
        if len({tensors[n].dtype for n in names}) != 1:
            raise ValueError("the projections of one mixer must be stored in one dtype to be stacked")
        # one stacked matrix on the device; every projection is a block of its rows (no second copy)
        self.stack = Linear(torch.cat([tensors[n].to(dev) for n in names], dim=0), self.rt)
        off = 0
        for name, n in self._stack_sizes():
            self.offsets[name] = off
            self.lin[name] = Linear(self.stack.weight[off:off + n], self.rt)
            off += n
        self.offsets["q"] = self.offsets["r"]
        self.proj_width = off
        # (the decay's second product reads 32-bit values behind the tanh and its inner size is tiny: the 32-bit kernels)
        self.w2 = Linear(tensors["w2"], self.rt, matrix_cores=False)
        self.w0 = tensors["w0"].to(dev).float().reshape(-1).contiguous()
        self.bonus = tensors["u"].to(dev).float().reshape(-1).contiguous()
        self.o = Linear(tensors["o"], self.rt)
        self.norm_weight = tensors["norm"].to(dev).float().contiguous()

    def weight_bytes(self) -> int:
        return self.stack.nbytes() + self.w2.nbytes() + self.o.nbytes() + 4 * (
            self.w0.numel() + self.bonus.numel() + self.norm_weight.numel())

    def input_projection(self):
        return None                           # (every projection reads a mix of its own)

    def _run(self, ctx, call, h, target, add: bool) -> None:
        ws, rows, W = ctx.ws, ctx.rows, self.width
        if h.shape[1] != len(self.inputs) * W:
            raise ValueError(f"wkv: the input must hold {len(self.inputs)} mixes of {W} elements side by side")
        nin, N = len(self.inputs), self.proj_width
        # (not where the product would first widen its rows into a buffer of the step's size)
        if rows <= self.FEW_ROWS and h.is_contiguous() and (self.stack.mfma or h.dtype == torch.float32):
            # Few rows: a launch costs more than its arithmetic, so the stacked matrix meets all the mixes of all the rows in
            # one product (the shifted rows read as rows * mixes rows of the model's width) and every projection is picked
            # from the rows of its own mix: row r's projection s lies at column s_mix * N + offset_s of a row of nin * N
            # columns.  A product's row does not depend on the rows beside it, so these are the bits of a product each.
            y = ws.buffer("recur_proj_few", N, torch.float32, rows=self.FEW_ROWS * nin)
            self.stack.store(ws, h.view(-1, W), y, rows * nin)
            y = y.view(self.FEW_ROWS, nin * N)
            at = {name: self.inputs.index("w" if name == "w1" else name) * N + self.offsets[name] for name, _ in self._stack_sizes()}
        else:
            y = ws.buffer("recur_proj", N, torch.float32)
            for name, n in self._stack_sizes():
                src = self.inputs.index("w" if name == "w1" else name) * W
                o = self.offsets[name]
                self.lin[name].store(ws, h[:, src:src + W], y[:, o:o + n], rows)
            at = dict(self.offsets)
        low = y[:, at["w1"]:at["w1"] + self.rank]
        ops.tanh_rows(low, rows)
        z = ws.buffer("wkv_decay_logits", self.heads * self.dim, torch.float32)
        self.w2.store(ws, low, z, rows)
        raw = ws.buffer("recur_out", self.heads * self.vdim, torch.float32)
        self._recur(ctx, call, y, z, 0, 0, self.w0, self.bonus, 0.0, raw, at=at)
        self._finish(ctx, y, raw, target, add, g_off=at["g"])

    def forward(self, ctx, call, h, residual) -> None:
        self._run(ctx, call, h, residual, True)

    def forward_out(self, ctx, call, h, out) -> None:
        self._run(ctx, call, h, out, False)


@register_mixer("retention")
class Retention(_MatrixMemoryMixer):
    """params: width, heads, dim, vdim, eps, decay (a number per head), position (PartSpec of a position encoding laid out
    in halves, or None).  tensors: q, k [heads*dim, width]; v, g [heads*vdim, width]; o [width, heads*vdim]."""

    mode = ops.RECUR_FIXED_DECAY
    gate_kind = ops.GATE_SILU
    per_head_norm_weight = False

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.kscale, self.qscale = float(self.dim) ** -0.5, 1.0      # (the keys carry the scale, behind their rotation)
        self.decay_values = [float(d) for d in params["decay"]]
        if len(self.decay_values) != self.heads or any(not 0.0 <= d <= 1.0 for d in self.decay_values):
            raise ValueError(f"retention: a decay in [0, 1] for each of the {self.heads} heads is needed")
        pos = params.get("position")
        self.position = None
        self.rot = 0
        if pos is not None:
            self.position = lookup(POSITION_ENCODINGS, "position encoding", pos.kind).shared(pos.params, runtime)
            if getattr(self.position, "layout", None) != "halves":
                raise ValueError(f"retention rotates halves of a head; position encoding '{pos.kind}' is laid out otherwise")
            self.rot = int(self.position.rotary_dim)
            if self.rot > self.dim:
                raise ValueError(f"retention: {self.rot} rotated elements in heads of {self.dim}")
        self.decay = self.cos = self.sin = None

    def _stack_sizes(self):
        hd, hv = self.heads * self.dim, self.heads * self.vdim
        return [("q", hd), ("k", hd), ("v", hv), ("g", hv)]

    def tensors(self):
        out = super().tensors()
        del out["norm"]                       # the read-out is divided by its root mean square and nothing else
        return out

    def bind(self, tensors) -> None:
        dev = self.rt.device
        self._bind_common(dict(tensors, norm=torch.ones(self.vdim)))
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=dev)
        if self.position is not None:
            self.cos, self.sin = self.position.tables()

    def weight_bytes(self) -> int:
        return self.proj.nbytes() + self.o.nbytes()

    def forward_out_projected(self, ctx, call, proj, out) -> None:
        self._run(ctx, call, None, out, False, projected=proj)

    def _run(self, ctx, call, h, target, add: bool, projected=None) -> None:
        y = projected if projected is not None else self._project(ctx, h)
        if self.rot:
            ops.rotate_halves_rows(y, (self.offsets["q"], self.offsets["k"]), self.heads, self.dim, self.rot, self.cos, self.sin,
                                   ctx.positions, ctx.rows)
        raw = ctx.ws.buffer("recur_out", self.heads * self.vdim, torch.float32)
        self._recur(ctx, call, y, None, 0, 0, self.decay, None, 0.0, raw, kscale=self.kscale)
        self._finish(ctx, y, raw, target, add)

    def forward(self, ctx, call, h, residual) -> None:
        self._run(ctx, call, h, residual, True)

    def forward_out(self, ctx, call, h, out) -> None:
        self._run(ctx, call, h, out, False)
