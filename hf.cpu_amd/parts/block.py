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
        norm_for(ops, parts["norm2"], parts["feed_forward"], x, h)
        ops.settle(x)
        parts["feed_forward"].forward(ops, step, h, x)


def norm_for(ops, norm, reader, x, out, rows=None):
    """``out = norm(x)`` for the part ``reader``: lazily if the norm can be and the reader reads ``out`` through
    ``ops.gemm`` alone."""
    if getattr(norm, "can_be_lazy", False) and getattr(reader, "lazy_input_ok", False):
        norm.forward(ops, x, out, rows, lazy=True)
    else:
        norm.forward(ops, x, out, rows)
