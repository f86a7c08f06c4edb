"""Arrangements of a layer's parts around the residual stream."""
from ..registry import register_part
from .base import Part


@register_part("block", "prenorm")
class PreNormBlock(Part):
    """``x += mixer(norm1(x)); x += feed_forward(norm2(x))`` (src/model.c:580-623):
    norms in front of each part, nothing after, the residual stream in fp32."""
    graph_safe = True


    def __init__(self, hidden_size, prefix=""):
        super().__init__(prefix)
        self.E = hidden_size

    def forward(self, ops, step, x, parts, caches, write_cache=True):
        """``parts``: norm1, mixer, norm2, feed_forward; ``caches``: the mixer's, under its name."""
        h = ops.scratch("normed", (x.shape[0], self.E), ops.act_dtype)
        norm_for(ops, parts["norm1"], parts["mixer"], x, h)      # also adds up a product the previous part deferred into x
        ops.settle(x)                          # (nothing left to do unless the norm could not)
        parts["mixer"].forward(ops, step, h, caches.get("mixer"), x, write_cache)
        if "feed_forward" not in parts:         # a layer may be its mixer alone
            return
        norm_for(ops, parts["norm2"], parts["feed_forward"], x, h)
        ops.settle(x)
        parts["feed_forward"].forward(ops, step, h, x)


@register_part("block", "parallel")
class ParallelBlock(Part):
    """``h = norm1(x); x += mixer(h) + feed_forward(h)``: one norm, both branches read its output, and both sums go
    into the fp32 stream. A layer without a feed-forward has the mixer alone."""
    graph_safe = True

    def __init__(self, hidden_size, prefix=""):
        super().__init__(prefix)
        self.E = hidden_size

    def forward(self, ops, step, x, parts, caches, write_cache=True):
        """``parts``: norm1, mixer and, if the layer has one, feed_forward; ``caches``: the mixer's, under its name."""
        h = ops.scratch("normed", (x.shape[0], self.E), ops.act_dtype)
        parts["norm1"].forward(ops, x, h)            # also adds up a product that the layer before deferred into x
        ops.settle(x)
        parts["mixer"].forward(ops, step, h, caches.get("mixer"), x, write_cache)
        ff = parts.get("feed_forward")
        if ff is not None:
            ff.forward(ops, step, h, x)


def norm_for(ops, norm, reader, x, out, rows=None):
    """``out = norm(x)`` for the part ``reader``: lazily if the norm can be and the reader reads ``out`` through
    ``ops.gemm`` alone."""
    if getattr(norm, "can_be_lazy", False) and getattr(reader, "lazy_input_ok", False):
        norm.forward(ops, x, out, rows, lazy=True)
    else:
        norm.forward(ops, x, out, rows)
