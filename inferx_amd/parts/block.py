"""Arrangement of a layer's parts.  `prenorm`:

    h += pending;  a = mixer(norm1(h));  h += a;  f = feed_forward(norm2(h));  pending = f

(reference: src/model/qwen2.cc:908-1051).  The residual stream h is float32 and
is updated inside the norm kernel, so each add is fused with the norm after it;
the last pending delta is added by the model's final norm.  A feed-forward that
says so gets norm2 unapplied (`LazyNorm`) and applies it in its first kernel.
"""
from __future__ import annotations

from .base import Block, LazyNorm, register_part


class PreNormBlock(Block):
    graph_safe = True
    part_kinds = {"mixer": "mixer", "feed_forward": "feed_forward", "mixer_norm": "norm", "feed_forward_norm": "norm"}

    def forward(self, ctx, h, pending, caches):
        x = self.mixer_norm.forward(ctx, h, pending)
        a = self.mixer.forward(ctx, x, caches.get("mixer"))
        if self.feed_forward.takes_lazy_norm:
            return self.feed_forward.forward(ctx, LazyNorm(self.feed_forward_norm, h, a))
        return self.feed_forward.forward(ctx, self.feed_forward_norm.forward(ctx, h, a))


register_part("block", "prenorm", PreNormBlock)
