"""Arrangements of norm, mixer and feed-forward in a block."""
from __future__ import annotations

from .base import Part, register_part


@register_part("block", "prenorm")
class PreNormBlock(Part):
    """h <- h + mixer(norm(h)); h <- h + ffn(norm(h)), with the sums carried in
    ``residual`` and made by the next norm (lite_llama/models/llama.py:138-162:
    the layer returns the feed-forward output and the residual without adding
    them; the next layer's first norm, or the final norm at :219, adds)."""

    def __init__(self, input_norm: Part, mixer: Part, post_norm: Part, feed_forward: Part):
        self.input_norm, self.mixer = input_norm, mixer
        self.post_norm, self.feed_forward = post_norm, feed_forward
        libs = ()
        for p in self.children().values():
            libs += tuple(p.kernel_libraries)
        self.kernel_libraries = tuple(dict.fromkeys(libs))

    def children(self):
        """Sub-parts by the role the model's naming scheme addresses them with."""
        return {"input_norm": self.input_norm, "mixer": self.mixer,
                "post_norm": self.post_norm, "feed_forward": self.feed_forward}

    def cache_spec(self):
        return self.mixer.cache_spec() if hasattr(self.mixer, "cache_spec") else None

    def forward(self, h, residual, ctx, cache):
        h, residual = self.input_norm.forward(h, residual)
        h = self.mixer.forward(h, ctx, cache)
        h, residual = self.post_norm.forward(h, residual)
        h = self.feed_forward.forward(h)
        return h, residual
