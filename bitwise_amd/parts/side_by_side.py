"""Several mixers side by side: all read the same input, each output is normed over the model width with a weight
vector of its own, and the mixer's output is the mean of the normed outputs.

    out = (1/n) sum_b  y_b / sqrt(mean(y_b^2) + eps) * w_b,      y_b = branch_b(h)

The branches are registered mixers of any kind; each keeps what it needs (pages of a cache, a slot of state) as it
would alone.  Towards the engine the combination is one mixer: its cache is the one branch's that has one (at most one
branch may page keys and values), its state slot holds the branches' states one behind the other."""

from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Tuple

import torch

from ..csrc import ops
from .base import MIXERS, CacheSpec, Mixer, PartSpec, StateSpec, TensorSpec, lookup, register_mixer
from .linear import Linear


@register_mixer("side_by_side")
class SideBySide(Mixer):
    """params: width, eps, branches: a list of (name, PartSpec of a mixer); a branch's tensors are its own behind
    ``<name>.``, and ``<name>.out`` [width] is the weight of the norm behind it."""

    SHARED_MAX_ROWS = 64       # steps of up to this many rows run the branches' first products as one

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.width, self.eps = int(params["width"]), float(params["eps"])
        self.names: List[str] = []
        self.branches: List[Mixer] = []
        for name, spec in params["branches"]:
            if not isinstance(spec, PartSpec):
                raise ValueError("side_by_side: every branch is a (name, PartSpec) pair")
            self.names.append(str(name))
            self.branches.append(lookup(MIXERS, "mixer", spec.kind)(spec.params, runtime))
        if not 1 <= len(self.branches) <= 4 or len(set(self.names)) != len(self.names):
            raise ValueError("side_by_side: one to four branches with names of their own")
        if sum(b.cache_spec() is not None for b in self.branches) > 1:
            raise ValueError("side_by_side: at most one branch may keep a paged cache")
        self.graph_safe = all(getattr(b, "graph_safe", False) for b in self.branches)
        self.launches_through_ops = all(getattr(b, "launches_through_ops", False) for b in self.branches)
        self.out_weights: List[torch.Tensor] = []
        self._post_weights: Dict[int, torch.Tensor] = {}      # 32-bit copies of the weights of norms that ride in the last launch
        # where each branch's state lies in the slot: (first element, elements), or None
        self.state_span: List[Optional[Tuple[int, int]]] = []
        at = 0
        for b in self.branches:
            ss = b.state_spec()
            if ss is None:
                self.state_span.append(None)
                continue
            if ss.dtype != "float32" or len(ss.shape) != 1:
                raise ValueError("side_by_side: the branches' states must be flat 32-bit vectors to share a slot")
            self.state_span.append((at, int(ss.shape[0])))
            at += int(ss.shape[0])
        self.state_elements = at

    # -- what the engine asks a mixer
    def tensors(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for name, b in zip(self.names, self.branches):
            for t, ts in b.tensors().items():
                out[f"{name}.{t}"] = ts
        for name in self.names:
            out[f"{name}.out"] = TensorSpec((self.width,), "norm")
        return out

    def bind(self, tensors) -> None:
        for name, b in zip(self.names, self.branches):
            b.bind({t: tensors[f"{name}.{t}"] for t in b.tensors()})
        self.out_weights = [tensors[f"{name}.out"].to(self.rt.device).float().contiguous() for name in self.names]
        # Branches whose whole reading of the input is one product each share one product: the matrices stacked (the
        # branches keep blocks of the stacked matrix, no copies), the branches read their columns of it.  A product's
        # column does not depend on the columns beside it, so these are the bits of a product each.
        self.shared_projection: Optional[Linear] = None
        self.shared_columns: List[Tuple[int, int]] = []
        firsts = [b.input_projection() for b in self.branches]
        if len(self.branches) > 1 and all(p is not None for p in firsts) and len({p.weight.dtype for p in firsts}) == 1 \
                and len({p.mfma for p in firsts}) == 1:
            self.shared_projection = Linear(torch.cat([p.weight for p in firsts], dim=0), self.rt)
            at = 0
            for b, p in zip(self.branches, firsts):
                n = p.out_features
                b.adopt_input_projection(self.shared_projection.weight[at:at + n])
                self.shared_columns.append((at, n))
                at += n

    def weight_bytes(self) -> int:
        # (a branch counts its block of the shared matrix as its own projection)
        return sum(b.weight_bytes() for b in self.branches) + 4 * self.width * len(self.branches)

    def cache_spec(self) -> Optional[CacheSpec]:
        for b in self.branches:
            cs = b.cache_spec()
            if cs is not None:
                return cs
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self.state_elements,), "float32") if self.state_elements else None

    def page_sizes(self):
        sizes = None
        for b in self.branches:
            s = b.page_sizes()
            if s is not None:
                sizes = tuple(s) if sizes is None else tuple(x for x in sizes if x in s)
        return sizes

    @property
    def prefix_reusable(self) -> bool:
        return all(b.prefix_reusable for b in self.branches)

    @property
    def run_ahead_safe(self) -> bool:
        return all(b.run_ahead_safe for b in self.branches)

    # -- the step
    def _branch_calls(self, ctx, call):
        """The call as each branch sees it: its own part of the state slot (a view), the cache if it is the one that pages."""
        def make():
            calls = []
            for b, span in zip(self.branches, self.state_span):
                state = None if span is None else call.state[:, span[0]:span[0] + span[1]]
                has_cache = b.cache_spec() is not None
                calls.append(dataclasses.replace(call, state=state, k_cache=call.k_cache if has_cache else None,
                                                 v_cache=call.v_cache if has_cache else None,
                                                 group=call.group if has_cache else -1))
            return calls
        return ctx.memo(("side_by_side_calls", id(self), call.index), make)

    def _branch_outputs(self, ctx, call, h, projected=None):
        ys = []
        # (steps of few rows, where a launch costs more than its arithmetic; a prompt portion's two products run faster apart
        # than one of their joint, odd number of columns: 2,048 rows of 2,576 + 6,144 columns took 0.14 ms longer as one)
        if projected is None and self.shared_projection is not None and ctx.rows <= self.SHARED_MAX_ROWS:
            projected = ctx.ws.buffer("side_by_side_projected", self.shared_projection.out_features, torch.float32)
            self.shared_projection.store(ctx.ws, h, projected, ctx.rows)
        for i, (b, sub) in enumerate(zip(self.branches, self._branch_calls(ctx, call))):
            y = ctx.ws.buffer(f"side_by_side_{i}", self.width, torch.float32)
            if projected is not None:
                at, n = self.shared_columns[i]
                b.forward_out_projected(ctx, sub, projected[:, at:at + n], y)
            else:
                b.forward_out(ctx, sub, h, y)
            ys.append(y)
        return ys

    def forward_out(self, ctx, call, h, out) -> None:
        ops.norm_mean(self._branch_outputs(ctx, call, h), self.out_weights, out, ctx.rows, self.eps)

    def _can_ride(self, norm) -> bool:
        from .norm import RMSNorm
        return type(norm) is RMSNorm and self.width <= ops.NORM_MEAN_ADD_MAX_WIDTH

    def _mean_add(self, ctx, ys, norm, x) -> None:
        w32 = self._post_weights.get(id(norm))
        if w32 is None:
            w32 = self._post_weights[id(norm)] = norm.weight.float().contiguous()       # (widening is exact)
        ops.norm_mean_add(ys, self.out_weights, self.eps, w32, norm.eps, norm.scale, x, ctx.rows)

    def forward_add_normed(self, ctx, call, h, norm, x) -> bool:
        """The norm behind the mixer rides in the launch that norms and averages the branches (the same bits)."""
        if not self._can_ride(norm):
            return False
        self._mean_add(ctx, self._branch_outputs(ctx, call, h), norm, x)
        return True

    def forward_between_norms(self, ctx, call, x, norm, norm_behind) -> bool:
        """Decode steps of few rows: the norm in front rides in the branches' one product (the bits of norm, then
        product), the norm behind in the launch that averages the branches."""
        from .norm import RMSNorm
        sp = self.shared_projection
        if not (sp is not None and self.rt.bf16 and sp.mfma and type(norm) is RMSNorm and self._can_ride(norm_behind)
                and ctx.rows <= self.SHARED_MAX_ROWS and ops.can_fuse_norm(ctx.rows, sp.weight, x)):
            return False
        projected = ctx.ws.buffer("side_by_side_projected", sp.out_features, torch.float32)
        ops.norm_gemm_bf16(x, norm.weight, norm.eps, sp.weight, projected, ctx.rows, ops.EPI_F32)
        self._mean_add(ctx, self._branch_outputs(ctx, call, None, projected), norm_behind, x)
        return True

    def forward(self, ctx, call, h, residual) -> None:
        y = ctx.ws.buffer("side_by_side_mean", self.width, torch.float32)
        self.forward_out(ctx, call, h, y)
        ops.add_(residual, y, ctx.rows)
