"""Arrangements of mixer, feed-forward and norms around the 32-bit residual stream."""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import Block, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """x += mixer(norm1(x)); x += feed_forward(norm2(x)) (src/model.cpp:281-305).  A layer may leave the feed-forward
    (and its norm) out."""

    roles = {"mixer_norm": "norm", "ffn_norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}
    optional_roles = ("ffn_norm", "feed_forward")
    graph_safe = True
    launches_through_ops = True

    def __init__(self, parts, runtime):
        super().__init__(parts, runtime)
        if (self.feed_forward is None) != (self.ffn_norm is None):
            raise ValueError("prenorm block: a feed-forward and its norm come together or not at all")

    def forward(self, ctx, call, x) -> None:
        if not self.mixer.forward_with_norm(ctx, call, x, self.mixer_norm, x):
            h = self.mixer_norm.forward(ctx, x)
            self.mixer.forward(ctx, call, h, x)
        if self.feed_forward is None:
            return
        if not self.feed_forward.forward_with_norm(ctx, x, self.ffn_norm, x):
            h = self.ffn_norm.forward(ctx, x)
            self.feed_forward.forward(ctx, h, x)


@register_block("parallel")
class ParallelBlock(Block):
    """x += mixer(norm1(x)) + feed_forward(norm2(x)), both read the same x; a layer may leave the feed-forward (and its
    norm) out.  A mixer norm with state of its own (a token shift) gets the call's ``block_state``."""

    roles = {"mixer_norm": "norm", "ffn_norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}
    optional_roles = ("ffn_norm", "feed_forward")
    graph_safe = True
    launches_through_ops = True

    def __init__(self, parts, runtime):
        super().__init__(parts, runtime)
        if (self.feed_forward is None) != (self.ffn_norm is None):
            raise ValueError("parallel block: a feed-forward and its norm come together or not at all")

    def state_spec(self):
        return self.mixer_norm.state_spec()

    def forward(self, ctx, call, x) -> None:
        # both branches' inputs are formed before either adds into x
        if call.block_state is not None:
            h = self.mixer_norm.forward(ctx, x, state=call.block_state)
        else:
            h = self.mixer_norm.forward(ctx, x, out_name="normed_mixer")
        if self.feed_forward is not None:
            # (the fused norm + product reads x before anything is added; the down projection adds afterwards)
            if not self.feed_forward.forward_with_norm(ctx, x, self.ffn_norm, x):
                h2 = self.ffn_norm.forward(ctx, x)
                self.feed_forward.forward(ctx, h2, x)
        self.mixer.forward(ctx, call, h, x)


@register_block("postnorm")
class PostNormBlock(Block):
    """x += norm1(mixer(x)); x += norm2(feed_forward(x)): the sublayers read the residual stream itself (in bfloat16
    mode its rounding, the only rounding between the stream and a sublayer's products), and each sublayer's output is
    normed on its way back into the stream.  A layer may leave the feed-forward (and its norm) out."""

    roles = {"mixer_norm": "norm", "ffn_norm": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}
    optional_roles = ("ffn_norm", "feed_forward")
    graph_safe = True
    launches_through_ops = True

    def __init__(self, parts, runtime):
        super().__init__(parts, runtime)
        if (self.feed_forward is None) != (self.ffn_norm is None):
            raise ValueError("postnorm block: a feed-forward and its norm come together or not at all")

    def _input(self, ctx, x):
        """The stream as the sublayer's products take it.  The kernel that adds a sublayer's normed output into the stream
        leaves the rounded copy behind (``forward_notes``: what parts tell later parts within one forward pass), so only
        a model's first layer converts."""
        if not self.rt.bf16:
            return x
        h = ctx.ws.buffer("stream_rounded", x.shape[1], torch.bfloat16)
        notes = getattr(ctx, "forward_notes", None)
        if notes is None or notes.get("stream_rounded") is not x:
            ops.convert(x, h, ctx.rows)
        return h

    def _add(self, ctx, norm, y, x) -> None:
        notes = getattr(ctx, "forward_notes", None)
        if self.rt.bf16 and notes is not None:
            norm.add_normed(ctx, y, x, rounded=ctx.ws.buffer("stream_rounded", x.shape[1], torch.bfloat16))
            notes["stream_rounded"] = x
        else:
            norm.add_normed(ctx, y, x)

    def forward(self, ctx, call, x) -> None:
        y = ctx.ws.buffer("sublayer_out", x.shape[1], torch.float32)
        self.mixer.forward_out(ctx, call, self._input(ctx, x), y)
        self._add(ctx, self.mixer_norm, y, x)
        if self.feed_forward is not None:
            h = self._input(ctx, x)
            notes = getattr(ctx, "forward_notes", None)
            rounded = ctx.ws.buffer("stream_rounded", x.shape[1], torch.bfloat16) if (self.rt.bf16 and notes is not None) else None
            if self.feed_forward.forward_add_normed(ctx, h, self.ffn_norm, x, rounded):
                if rounded is not None:
                    notes["stream_rounded"] = x
            else:
                self.feed_forward.forward_out(ctx, h, y)
                self._add(ctx, self.ffn_norm, y, x)


@register_block("sandwich")
class SandwichBlock(Block):
    """x += norm1b(mixer(norm1(x))); x += norm2b(feed_forward(norm2(x))): a norm in front of each sublayer and another
    behind it, on its way into the stream (a factor on that second norm, its ``scale``, weighs the sublayer against the
    stream).  A layer may leave the feed-forward (and its two norms) out.  A mixer norm with state of its own (a token
    shift) gets the call's ``block_state``."""

    roles = {"mixer_norm": "norm", "mixer_post_norm": "norm", "ffn_norm": "norm", "ffn_post_norm": "norm", "mixer": "mixer",
             "feed_forward": "feed_forward"}
    optional_roles = ("ffn_norm", "ffn_post_norm", "feed_forward")
    graph_safe = True
    launches_through_ops = True

    def __init__(self, parts, runtime, params=None):
        super().__init__(parts, runtime, params)
        if len({self.feed_forward is None, self.ffn_norm is None, self.ffn_post_norm is None}) != 1:
            raise ValueError("sandwich block: a feed-forward and its two norms come together or not at all")

    def state_spec(self):
        return self.mixer_norm.state_spec()

    def forward(self, ctx, call, x) -> None:
        if call.block_state is None and self.mixer.forward_between_norms(ctx, call, x, self.mixer_norm, self.mixer_post_norm):
            h = None
        elif call.block_state is not None:
            h = self.mixer_norm.forward(ctx, x, state=call.block_state)
        else:
            h = self.mixer_norm.forward(ctx, x)
        if h is not None and not self.mixer.forward_add_normed(ctx, call, h, self.mixer_post_norm, x):
            y = ctx.ws.buffer("sublayer_out", x.shape[1], torch.float32)
            self.mixer.forward_out(ctx, call, h, y)
            self.mixer_post_norm.add_normed(ctx, y, x)
        if self.feed_forward is None:
            return
        h = self.ffn_norm.forward(ctx, x)
        if not self.feed_forward.forward_add_normed(ctx, h, self.ffn_post_norm, x):
            y = ctx.ws.buffer("sublayer_out", x.shape[1], torch.float32)
            self.feed_forward.forward_out(ctx, h, y)
            self.ffn_post_norm.add_normed(ctx, y, x)
