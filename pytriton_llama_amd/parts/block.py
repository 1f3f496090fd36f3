"""Arrangements of norm, mixer and feed-forward in a block."""
from __future__ import annotations

from .base import Part, as_tensor, register_part, run_norm


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

    def work_lists(self):
        """The work lists its parts want (parts.base.WorkList)."""
        lists = ()
        for p in self.children().values():
            if hasattr(p, "work_lists"):
                lists += tuple(p.work_lists())
        return tuple(dict.fromkeys(lists))

    can_defer_output = True

    @property
    def takes_pending_product(self) -> bool:
        """Whether the block before this one may leave its last product to this block's first
        norm (parts/base.py): what the model asks when it runs two blocks in a row."""
        return bool(getattr(self.input_norm, "takes_pending_product", False))

    def make_decode_copies(self) -> int:
        return sum(p.make_decode_copies() for p in self.children().values()
                   if hasattr(p, "make_decode_copies"))

    @property
    def graph_capturable(self) -> bool:
        return all(getattr(p, "graph_capturable", True) for p in self.children().values())

    def forward(self, h, residual, ctx, cache, defer_output: bool = False):
        """``h`` may be pending work of the block before (parts/base.py); with ``defer_output``
        the feed-forward may leave its last product to whoever normalises next."""
        mixer, ffn = self.mixer, self.feed_forward
        h, residual = run_norm(self.input_norm, h, residual, mixer)
        if not getattr(mixer, "takes_pending_scale", False):
            h = as_tensor(h)
        if (getattr(mixer, "can_defer_output", False)
                and getattr(self.post_norm, "takes_pending_product", False)):
            h = mixer.forward(h, ctx, cache, defer_output=True)
        else:
            h = mixer.forward(h, ctx, cache)
        h, residual = run_norm(self.post_norm, h, residual, ffn)
        if not getattr(ffn, "takes_pending_scale", False):
            h = as_tensor(h)
        if defer_output and getattr(ffn, "can_defer_output", False):
            h = ffn.forward(h, defer_output=True)
        else:
            h = ffn.forward(h)
        return h, residual
