"""Arrangements of a layer's parts.

``pre_norm`` is the reference's block (``src/model/qwen3.cpp:216-239``):
``x += mixer(norm(x)); x += feed_forward(norm(x))`` with the norms named
``pre_mixer`` and ``pre_feed_forward`` in the layer's spec and nothing applied
to the sub-layer outputs. A layer that has only one of the two parts runs that
half alone (and needs that half's norm only).

``sandwich_norm`` norms both sides of each sub-layer: ``x += post_mixer(mixer(pre_mixer(x)))`` and then
``x += post_feed_forward(feed_forward(pre_feed_forward(x)))``. The sub-layers are asked for their result instead of
adding it (``forward(..., residual=None)``); the norm over the result, the addition to the stream and the norm
that the stream meets next run as one kernel where the norms can (``Norm.add_normed``).
"""

from __future__ import annotations

import torch

from ..errors import InvalidArgument
from .base import Block, StepContext, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True
    NORMS = ("pre_mixer", "pre_feed_forward")

    def forward(self, ctx: StepContext, x: torch.Tensor, layer, cache) -> None:
        if layer.mixer is not None:
            h = self.normed(ctx, layer.norms["pre_mixer"], x, consumer=layer.mixer)
            layer.mixer.forward(ctx, h, cache, x)
        if layer.feed_forward is not None:
            h = self.normed(ctx, layer.norms["pre_feed_forward"], x, consumer=layer.feed_forward)
            layer.feed_forward.forward(ctx, h, x)

    @classmethod
    def check_layer(cls, layer) -> None:
        needed = [n for n, part in zip(cls.NORMS, (layer.mixer, layer.feed_forward)) if part is not None]
        if not needed:
            raise InvalidArgument("a pre_norm block needs a mixer, a feed-forward or both")
        missing = [n for n in needed if n not in layer.norms]
        if missing:
            raise InvalidArgument(f"a pre_norm block needs the norms {', '.join(needed)}; missing {', '.join(missing)}")


@register_part("block", "sandwich_norm")
class SandwichNormBlock(Block):
    capturable = True
    replayable = True
    MIXER_NORMS = ("pre_mixer", "post_mixer")
    FEED_FORWARD_NORMS = ("pre_feed_forward", "post_feed_forward")

    @staticmethod
    def _result(ctx: StepContext, part, run):
        """The sub-layer's result: its own (``residual=None``), or for a part that can only add, what it adds to zeros."""
        if getattr(part, "returns_result", False):
            return run(None)
        zeros = ctx.scratch("block.sublayer_result", (ctx.num_tokens, part.hidden), torch.float32)
        zeros.zero_()
        run(zeros)
        ctx.settle()
        return zeros

    @staticmethod
    def _place(ctx: StepContext, post, y, x: torch.Tensor, following=None):
        if hasattr(post, "add_normed"):
            fused = following if isinstance(following, type(post)) else None
            h = post.add_normed(ctx, y, x, next_norm=fused)
            return h
        if not isinstance(y, torch.Tensor) or y.dim() != 2:
            raise InvalidArgument("this norm takes a sub-layer's result as plain rows only")
        x.add_(post.forward(ctx, y, out_name="norm.post", out_dtype=torch.float32))
        return None

    def forward(self, ctx: StepContext, x: torch.Tensor, layer, cache) -> None:
        norms = layer.norms
        h = None
        if layer.mixer is not None:
            h = self.normed(ctx, norms["pre_mixer"], x)
            y = self._result(ctx, layer.mixer, lambda residual: layer.mixer.forward(ctx, h, cache, residual))
            following = norms["pre_feed_forward"] if layer.feed_forward is not None else None
            h = self._place(ctx, norms["post_mixer"], y, x, following)
        if layer.feed_forward is not None:
            if h is None:
                h = self.normed(ctx, norms["pre_feed_forward"], x)
            rows = h
            y = self._result(ctx, layer.feed_forward, lambda residual: layer.feed_forward.forward(ctx, rows, residual))
            self._place(ctx, norms["post_feed_forward"], y, x)

    @classmethod
    def check_layer(cls, layer) -> None:
        needed = (cls.MIXER_NORMS if layer.mixer is not None else ()) + \
            (cls.FEED_FORWARD_NORMS if layer.feed_forward is not None else ())
        if not needed:
            raise InvalidArgument("a sandwich_norm block needs a mixer, a feed-forward or both")
        missing = [n for n in needed if n not in layer.norms]
        if missing:
            raise InvalidArgument(f"a sandwich_norm block needs the norms {', '.join(needed)}; missing {', '.join(missing)}")
