"""Block arrangements.

'sandwich' is the block of simply/model_lib.py:2659-2708 with use_pre_ln and use_post_ln:
  h += post_mixer(mixer(pre_mixer(h)));  h += post_ffn(ffn(pre_ffn(h)))
The residual stream h is float32; each residual sum is fused with the norm before it and the
norm after it where those are RMSNorms.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import BLOCKS
from .base import Block, PendingNorm
from .norm import NoNorm

#: stands for "no norm follows": the kernel of the last residual sum then hands the stream on in the activation type
_HAND_ON = NoNorm()


@BLOCKS.register("sandwich")
class SandwichBlock(Block):
    """A layer may have no feed-forward (its step and norms are then left out), and parts that update the residual
    stream themselves may follow (`extras`)."""

    NORM_NAMES = ("pre_mixer", "post_mixer", "pre_ffn", "post_ffn")
    takes_extras = True

    def __init__(self, mixer, feed_forward, norms, extras=()):
        super().__init__(mixer, feed_forward, norms, extras)
        missing = [n for n in self.NORM_NAMES[:4 if feed_forward is not None else 2] if n not in self.norms]
        if missing:
            raise ValueError(f"sandwich block: norms missing: {missing}")

    def first_norm(self):
        return self.norms["pre_mixer"]

    def forward(self, h, ctx, cache, normed, next_norm):
        n = self.norms
        if ctx.dtype == torch.bfloat16 and ctx.positions.is_cuda and ctx.num_tokens <= ops.few_rows_limit():
            return self._forward_few_rows(h, ctx, cache, normed, next_norm)
        if isinstance(normed, PendingNorm):
            normed, h = normed.materialize(), normed.residual
        if normed is None:
            normed = n["pre_mixer"].forward(h, ctx.dtype)
        # (a part's last product may leave the sum of its cuts of K to the norm behind it, where both can)
        def defer(part, norm):
            both = part.defers_sum and getattr(norm, "adds_partial_sums", False) and ctx.dtype == torch.bfloat16
            return {"defer_sum": True} if both else {}

        # (parts behind the feed-forward change the stream once more: the next block's norm comes after them; they read
        # the stream in the activation type, which the kernel of the last sum hands on)
        after = _HAND_ON if self.extras else next_norm
        y = self.mixer.forward(normed, ctx, cache, **defer(self.mixer, n["post_mixer"]))
        if self.feed_forward is None:
            normed_next = n["post_mixer"].add_into(h, y, after, ctx.dtype)
        else:
            normed = n["post_mixer"].add_into(h, y, n["pre_ffn"], ctx.dtype)
            y = self.feed_forward.forward(normed, ctx, **defer(self.feed_forward, n["post_ffn"]))
            normed_next = n["post_ffn"].add_into(h, y, after, ctx.dtype)
        if self.extras:
            for k, part in enumerate(self.extras):
                part.forward(h, ctx, x=normed_next if k == 0 else None)
            normed_next = next_norm.forward(h, ctx.dtype) if next_norm is not None else None
        return h, normed_next

    def _forward_few_rows(self, h, ctx, cache, normed, next_norm):
        """The same block for a handful of rows (decoding): every "residual sum, norm" between two parts is handed
        on as a `PendingNorm`, which the next part's first product computes in its own kernel."""
        n = self.norms

        def give(part, x):
            if isinstance(x, PendingNorm) and not part.accepts_pending:
                return x.materialize()
            return x

        x = normed if normed is not None else PendingNorm(h, None, None, n["pre_mixer"], ctx.dtype)
        y = self.mixer.forward(give(self.mixer, x), ctx, cache)
        if isinstance(x, PendingNorm):
            h = x.settle()
        last = "post_mixer"
        if self.feed_forward is not None:
            x = PendingNorm(h, y, n["post_mixer"], n["pre_ffn"], ctx.dtype)
            y = self.feed_forward.forward(give(self.feed_forward, x), ctx)
            h = x.settle()
            last = "post_ffn"
        if not self.extras:
            return h, PendingNorm(h, y, n[last], next_norm, ctx.dtype)
        handed = n[last].add_into(h, y, _HAND_ON, ctx.dtype)
        for k, part in enumerate(self.extras):
            part.forward(h, ctx, x=handed if k == 0 else None)
        return h, PendingNorm(h, None, None, next_norm, ctx.dtype)


@BLOCKS.register("post_norm")
class PostNormBlock(Block):
    """h += post_mixer(mixer(h));  h += post_ffn(ffn(h)): the parts read the residual stream itself (in the
    activation type), only what they return is normed.  A layer may have no feed-forward; then the second step is
    left out.  A constant that scales what is added (a residual multiplier) is the norms' own factor.  Norms: 'input'
    (what stands in front of both parts: usually the norm that is none), 'post_mixer', and 'post_ffn' if there is a
    feed-forward."""

    def __init__(self, mixer, feed_forward, norms):
        super().__init__(mixer, feed_forward, norms)
        wanted = ("input", "post_mixer") + (("post_ffn",) if feed_forward is not None else ())
        missing = [n for n in wanted if n not in self.norms]
        if missing:
            raise ValueError(f"post_norm block: norms missing: {missing}")

    def first_norm(self):
        return self.norms["input"]

    def forward(self, h, ctx, cache, normed, next_norm):
        n = self.norms
        if isinstance(normed, PendingNorm):
            normed, h = normed.materialize(), normed.residual
        if normed is None:
            normed = n["input"].forward(h, ctx.dtype)
        y = self.mixer.forward(normed, ctx, cache)
        if self.feed_forward is None:
            return h, n["post_mixer"].add_into(h, y, next_norm, ctx.dtype)
        normed = n["post_mixer"].add_into(h, y, n["input"], ctx.dtype)
        y = self.feed_forward.forward(normed, ctx)
        return h, n["post_ffn"].add_into(h, y, next_norm, ctx.dtype)


@BLOCKS.register("pre_norm")
class PreNormBlock(Block):
    """h += mult * mixer(pre_mixer(h));  h += mult * ffn(pre_ffn(h)): the parts read normed input, what they return is
    added as it is, times a constant (`mult`, a residual multiplier).  A layer may have no feed-forward; then the
    second step is left out.  Each sum runs in one kernel with the norm in front of the next part where that is an
    RMSNorm."""

    def __init__(self, mixer, feed_forward, norms, mult: float = 1.0):
        super().__init__(mixer, feed_forward, norms)
        self.mult = float(mult)
        wanted = ("pre_mixer",) + (("pre_ffn",) if feed_forward is not None else ())
        missing = [n for n in wanted if n not in self.norms]
        if missing:
            raise ValueError(f"pre_norm block: norms missing: {missing}")

    def first_norm(self):
        return self.norms["pre_mixer"]

    def _add(self, h, y, norm, dtype):
        """h += mult * y; returns norm(h), or None without a norm."""
        if norm is not None and getattr(norm, "fusable_rms", False):
            return ops.residual_add_next_norm(y, h, norm.scale, eps=norm.eps, plus_one=norm.scale_plus_one,
                                              mult=self.mult, out_dtype=dtype)
        ops.residual_add_norm(y, h, mult=self.mult)
        return norm.forward(h, dtype) if norm is not None else None

    def forward(self, h, ctx, cache, normed, next_norm):
        n = self.norms
        if isinstance(normed, PendingNorm):
            normed, h = normed.materialize(), normed.residual
        if normed is None:
            normed = n["pre_mixer"].forward(h, ctx.dtype)
        y = self.mixer.forward(normed, ctx, cache)
        if self.feed_forward is None:
            return h, self._add(h, y, next_norm, ctx.dtype)
        normed = self._add(h, y, n["pre_ffn"], ctx.dtype)
        y = self.feed_forward.forward(normed, ctx)
        return h, self._add(h, y, next_norm, ctx.dtype)
