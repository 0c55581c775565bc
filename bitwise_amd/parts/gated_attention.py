"""Causal grouped-query attention with a short convolution behind its projections, unit-normed rotated queries and
keys, a sink in the softmax and a gate on its output; a layer may read the keys and values another layer cached.

    q, k, v = conv(W_q h), conv(W_k h), conv(W_v h)       a causal convolution over `taps` tokens per channel
    q, k    = unit(rot(q)), unit(rot(k))                   pairs (2i, 2i+1) of the first rot elements turned by the
                                                           position's angles, then x / sqrt(mean(x^2) + eps) per head
    p_j     = exp(s_j) / (exp(sink) + sum_i exp(s_i))      s_j = scale * q . k_j over the keys j <= the query's position
    out     = W_o ((sum_j p_j v_j) * sigmoid(W_g h))

Every step is switched by a parameter, so that another design can take what it needs: ``conv`` (taps; 0 or 1 with no
convolution tensor: none), ``qk_norm``, ``sink`` (None, or a number that every head uses), ``gate``, ``shared_kv``
(no key and value tensors: the call reads the cache of the layer the schedule names), query/key size ``dim`` and value
size ``vdim`` (the cache's head size is the larger of the two, rounded up to what the attention kernels take; the
padding is zeros).  Further switches:

    position None          no rotation: positions do not enter the scores
    qk_norm "whole"        q and k are normed over their whole projection, all heads at once, with learned weights
                           (tensors q.norm, k.norm): x / sqrt(mean(x^2) + eps) * w
    softcap c              s_j <- c tanh(s_j / c) before the softmax
    chunk C                the query at position i sees key j <= i only if floor(i / C) = floor(j / C), positions counted
                           from the request's first token (not together with a window)
    v_mix "source"/"mix"   the first such layer of a model keeps its values of the step's rows ("source"); a later one
                           ("mix") caches v <- (1 - lambda) v + lambda v_source, lambda the tensor ``vmix`` (one number)
    position layout        a position encoding laid out in "halves" turns element i together with element i + rot/2
    values "keys"          there is no value projection: a token's values are its keys as projected, before rotation
    sink "learned"         the sink is a tensor ``sink`` [heads], a number per head
    gate "head"            the gate is one number per head, sigmoid(W_g h) with W_g [heads, width]
    window W               the query at position i sees the keys i - W + 1 .. i
  The last taps - 1 projected rows of a request are its state.  Convolution, rotation, norms, scores
and softmax are 32-bit in both modes; the cache, the queries and the gated output have the mode's activation dtype.
"""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from .attention import attend_bf16, attend_f32
from .base import CacheSpec, Mixer, StateSpec, TensorSpec, lookup, register_mixer, POSITION_ENCODINGS
from .linear import Linear


def max_seq_rows(ctx) -> int:
    """The most rows one request brings in this step."""
    if getattr(ctx, "one_row_per_request", False):
        return 1
    return ctx.memo(("max_seq_rows",), lambda: max(len(s.tokens) for s in ctx.segments))


@register_mixer("gated_attention")
class GatedAttention(Mixer):
    """params: width, heads, kv_heads, dim, vdim, scale, eps, conv (taps), qk_norm, sink (None, a number or "learned"), gate
    (False, True or "head"), values ("own" or "keys"), shared_kv, window, softcap, chunk, v_mix, position (PartSpec of a
    position encoding with the layout "pairs" or "halves").
    tensors: q, k, v [heads*dim | kv_heads*dim | kv_heads*vdim, width] (no v where the values are the keys); q.conv, k.conv,
    v.conv [channels, taps]; g [heads*vdim, width] (a gate a head: [heads, width]); sink [heads] if learned;
    o [width, heads*vdim]."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        p = params
        self.width, self.heads, self.kv_heads = int(p["width"]), int(p["heads"]), int(p["kv_heads"])
        self.dim, self.vdim = int(p["dim"]), int(p["vdim"])
        self.scale, self.eps = float(p["scale"]), float(p.get("eps", 0.0))
        self.taps = int(p.get("conv") or 0)
        self.whole_norm = p.get("qk_norm") == "whole"
        self.qk_norm, self.gate, self.shared_kv = bool(p.get("qk_norm", False)), bool(p.get("gate", False)), bool(p.get("shared_kv", False))
        self.head_gate = p.get("gate") == "head"
        self.values_are_keys = p.get("values") == "keys"
        if p.get("values") not in (None, "own", "keys"):
            raise ValueError(f"gated_attention: values are 'own' or 'keys', not {p.get('values')!r}")
        if self.values_are_keys and (self.dim != self.vdim or self.shared_kv or self.whole_norm or int(p.get("conv") or 0) > 1):
            raise ValueError("gated_attention: values that are the keys have the keys' size, in a layer with keys of its own, "
                             "without a convolution or a norm over whole projections")
        self.softcap = float(p.get("softcap") or 0.0)
        self.chunk = int(p.get("chunk") or 0)
        self.v_mix = p.get("v_mix") or None
        if self.v_mix not in (None, "source", "mix"):
            raise ValueError(f"gated_attention: v_mix is 'source' or 'mix', not {self.v_mix!r}")
        if self.v_mix is not None and (self.shared_kv or not self.whole_norm):
            raise ValueError("gated_attention: values are mixed by the kernel that norms whole projections, in layers with values of their own")
        if self.softcap < 0 or self.chunk < 0 or (self.chunk and p.get("window")):
            raise ValueError("gated_attention: a soft cap and a chunk are positive; a chunk does not go with a window")
        self.learned_sink = p.get("sink") == "learned"
        self.sink_value: Optional[float] = None if p.get("sink") is None or self.learned_sink else float(p["sink"])
        self.window: Optional[int] = p.get("window")
        if self.heads % self.kv_heads:
            raise ValueError(f"gated_attention: {self.heads} heads are no multiple of {self.kv_heads} kv heads")
        if not self.scale > 0:
            raise ValueError("gated_attention: the score scale must be positive")
        if self.taps > ops.CONV_MAX_TAPS:
            raise ValueError(f"gated_attention: a convolution over {self.taps} tokens; the kernel takes up to {ops.CONV_MAX_TAPS}")
        need = max(self.dim, self.vdim)
        fits = [d for d in ops.HEAD_DIMS if d >= need]
        if not fits:
            raise ValueError(f"gated_attention: heads of {need} elements; the attention kernels take up to {ops.HEAD_DIMS[-1]}")
        self.head_size = fits[0]                       # the cache's head size
        pos = p.get("position")
        self.position = None
        self.rot = 0
        if pos is not None:
            self.position = lookup(POSITION_ENCODINGS, "position encoding", pos.kind).shared(pos.params, runtime)
            if getattr(self.position, "layout", None) not in ("pairs", "halves"):
                raise ValueError(f"gated_attention rotates neighbouring pairs or halves; position encoding '{pos.kind}' is laid out otherwise")
            self.rot = int(self.position.rotary_dim)
        self.halves = getattr(self.position, "layout", None) == "halves"
        if self.whole_norm and self.rot:
            raise ValueError("gated_attention: the norm over whole projections comes without rotation")
        if self.rot > self.dim:
            raise ValueError(f"gated_attention: {self.rot} rotated elements in heads of {self.dim}")
        self.q_ch = self.heads * self.dim
        self.kv_ch = 0 if self.shared_kv else self.kv_heads * (self.dim + (0 if self.values_are_keys else self.vdim))
        self.conv_ch = self.q_ch + self.kv_ch
        self.g_ch = (self.heads if self.head_gate else self.heads * self.vdim) if self.gate else 0
        self.proj: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.conv_w = self.sink = self.cos = self.sin = None
        self.q_norm_w = self.k_norm_w = self.mix_w = None

    def tensors(self) -> Dict[str, TensorSpec]:
        out = {"q": TensorSpec((self.q_ch, self.width))}
        if not self.shared_kv:
            out["k"] = TensorSpec((self.kv_heads * self.dim, self.width))
            if not self.values_are_keys:
                out["v"] = TensorSpec((self.kv_heads * self.vdim, self.width))
        if self.learned_sink:
            out["sink"] = TensorSpec((self.heads,), "bias")
        if self.taps >= 1:
            out["q.conv"] = TensorSpec((self.q_ch, self.taps), "conv")
            if not self.shared_kv:
                out["k.conv"] = TensorSpec((self.kv_heads * self.dim, self.taps), "conv")
                out["v.conv"] = TensorSpec((self.kv_heads * self.vdim, self.taps), "conv")
        if self.whole_norm:
            out["q.norm"] = TensorSpec((self.q_ch,), "norm")
            if not self.shared_kv:
                out["k.norm"] = TensorSpec((self.kv_heads * self.dim,), "norm")
        if self.v_mix is not None:
            out["vmix"] = TensorSpec((), "unit_interval")      # (read by "mix" layers; a "source" layer's is stored and unused)
        if self.gate:
            out["g"] = TensorSpec((self.g_ch, self.width))
        out["o"] = TensorSpec((self.width, self.heads * self.vdim))
        return out

    def bind(self, tensors) -> None:
        dev = self.rt.device
        if self.position is not None:
            self.cos, self.sin = self.position.tables()
        else:
            self.cos = self.sin = torch.zeros(1, dtype=torch.float32, device=dev)      # (never read: nothing is rotated)
        if self.whole_norm:
            self.q_norm_w = tensors["q.norm"].to(dev).float().contiguous()            # (widening is exact)
            self.k_norm_w = self.q_norm_w if self.shared_kv else tensors["k.norm"].to(dev).float().contiguous()
        if self.v_mix == "mix":
            self.mix_w = tensors["vmix"].to(dev).float().reshape(1).contiguous()
        names = ["q"] + ([] if self.shared_kv else (["k"] if self.values_are_keys else ["k", "v"])) + (["g"] if self.gate else [])
        stack = [tensors[n] for n in names]
        if len({t.dtype for t in stack}) != 1:
            raise ValueError("the projections of one mixer must be stored in one dtype to be stacked")
        self.proj = Linear(torch.cat(stack, dim=0), self.rt)
        self.o = Linear(tensors["o"], self.rt)
        if self.taps >= 1:
            cn = ["q.conv"] + ([] if self.shared_kv else ["k.conv", "v.conv"])
            self.conv_w = torch.cat([tensors[n].to(dev).float() for n in cn], dim=0).contiguous()      # (widening is exact)
        if self.learned_sink:
            self.sink = tensors["sink"].to(dev).float().contiguous()
        elif self.sink_value is not None:
            self.sink = torch.full((self.heads,), self.sink_value, dtype=torch.float32, device=dev)

    def weight_bytes(self) -> int:
        return self.proj.nbytes() + self.o.nbytes() + (0 if self.conv_w is None else self.conv_w.numel() * 4)

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(self.kv_heads, self.head_size, self.window)

    def page_sizes(self):
        return ops.PAGE_SIZES

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec(((self.taps - 1) * self.conv_ch,), "float32") if self.taps > 1 else None

    def input_projection(self):
        # (the plain arrangement only: rotation, cache write and gate read the product's columns by their stride)
        return self.proj if self.proj is not None and self.taps < 1 and not self.whole_norm else None

    def adopt_input_projection(self, weight) -> None:
        self.proj = Linear(weight, self.rt)

    def forward_out_projected(self, ctx, call, proj, out) -> None:
        self._run(ctx, call, None, out, False, projected=proj)

    def _run(self, ctx, call, h, target, add: bool, normed_from=None, projected=None) -> None:
        """``normed_from`` = (x, norm) instead of ``h``: the norm rides in the projections' product.  ``projected``: the
        projections' 32-bit sums, already made (columns of a wider product)."""
        rt, ws, rows = self.rt, ctx.ws, ctx.rows
        if self.shared_kv == bool(call.writes_cache):
            raise ValueError("gated_attention: a layer with keys and values of its own writes its cache, one without reads another's")
        proj = projected if projected is not None else ws.buffer("gattn_proj", self.proj.out_features, torch.float32)
        if projected is not None:
            pass
        elif normed_from is not None:
            x, norm = normed_from
            ops.norm_gemm_bf16(x, norm.weight, norm.eps, self.proj.weight, proj, rows, ops.EPI_F32)
        else:
            self.proj.store(ws, h, proj, rows)
        src = proj
        if self.taps >= 1:
            src = ws.buffer("gattn_conv", self.conv_ch, torch.float32)
            ops.causal_conv(proj, self.conv_w, None, call.state, ctx.seq_rows, ctx.slots, ctx.positions, ctx.nseq,
                            max_seq_rows(ctx), src)
        hs = self.head_size
        q = ws.buffer("gattn_q", self.heads * hs, rt.act_dtype)
        if self.whole_norm:
            v_first = v_keep = None
            if self.v_mix is not None:
                # the source layer's values of this step's rows, as projected: what the layers tell each other within a pass
                notes = ctx.forward_notes
                key = ("v_mix_source", self.kv_heads * self.vdim)
                if self.v_mix == "source":
                    v_keep = notes[key] = ws.buffer("v_mix_source", self.kv_heads * self.vdim, torch.float32)
                else:
                    v_first = notes.get(key)
                    if v_first is None:
                        raise ValueError("gated_attention: a layer mixes values before any layer has kept its own")
            ops.whole_norm_kv(src, ctx.positions, ctx.row_seq, ctx.block_tables[call.group], self.q_norm_w, self.k_norm_w, self.eps,
                              q, call.k_cache, call.v_cache, rows, self.heads, self.kv_heads, self.dim, self.vdim, hs,
                              ws.page_size, call.writes_cache, v_first=v_first, mix=self.mix_w, v_keep=v_keep)
        else:
            ops.pair_rope_unit(src, ctx.positions, ctx.row_seq, ctx.block_tables[call.group], self.cos, self.sin, q, call.k_cache,
                               call.v_cache, rows, self.heads, self.kv_heads, self.dim, self.vdim, hs, self.rot, ws.page_size,
                               self.qk_norm, self.eps, not self.shared_kv, call.writes_cache, halves=self.halves,
                               values_are_keys=self.values_are_keys)
        av = ws.buffer("gattn_av", self.heads * hs, rt.act_dtype)
        attend = attend_bf16 if rt.bf16 else attend_f32
        attend(ctx, call, q, av, self.heads, self.kv_heads, hs, int(self.window or 0), self.scale, sink=self.sink,
               chunk=self.chunk, softcap=self.softcap)
        if self.gate or hs != self.vdim:
            act = ws.buffer("gattn_gated", self.heads * self.vdim, rt.act_dtype)
            if self.gate:
                ops.gate_mul(av, hs, proj[:, self.conv_ch:], act, rows, self.heads, self.vdim, per_head=self.head_gate)
            else:
                act.view(-1, self.heads, self.vdim)[:rows].copy_(av.view(-1, self.heads, hs)[:rows, :, :self.vdim])
        else:
            act = av
        if add:
            self.o.add_into(ws, act, target, rows)
        else:
            self.o.store(ws, act, target, rows)

    def forward(self, ctx, call, h, residual) -> None:
        self._run(ctx, call, h, residual, True)

    def forward_with_norm(self, ctx, call, x, norm, residual) -> bool:
        """Decode steps of few rows: the norm in front of the mixer rides in the stacked projections' product (the bits of
        norm, then product)."""
        from .norm import RMSNorm
        if not (self.rt.bf16 and type(norm) is RMSNorm and self.proj.mfma and self.proj.bias is None
                and ops.can_fuse_norm(ctx.rows, self.proj.weight, x)):
            return False
        self._run(ctx, call, None, residual, True, normed_from=(x, norm))
        return True

    def forward_out(self, ctx, call, h, out) -> None:
        self._run(ctx, call, h, out, False)
