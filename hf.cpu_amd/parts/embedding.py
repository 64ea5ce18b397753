"""Token embedding and the output head."""
from ..registry import register_part
from .base import ParamSpec, Part


@register_part("embedding", "lookup")
class Embedding(Part):
    """``x[t, :] = table[token[t], :]`` without scaling (src/model.c:566-571)."""
    graph_safe = True


    def __init__(self, vocab_size, hidden_size, prefix=""):
        super().__init__(prefix)
        self.V, self.E = vocab_size, hidden_size
        self.table = None

    def param_specs(self):
        return [ParamSpec(self.prefix + "weight", (self.V, self.E))]

    def bind(self, params, ops):
        self.table = params[self.prefix + "weight"]

    def forward(self, ops, step, out_x):
        with ops.section("embed"):
            ops.embed(self.table, step.tokens, out_x)


@register_part("head", "linear")
class LinearHead(Part):
    """``logits = W h`` in fp32, no bias (src/model.c:633-635). With ``tied`` the
    matrix is the embedding table unless the checkpoint holds one of its own, which
    then wins (src/model.c:156-158)."""
    graph_safe = True
    lazy_input_ok = True


    def __init__(self, vocab_size, hidden_size, tied, tied_to="", prefix=""):
        super().__init__(prefix)
        self.V, self.E = vocab_size, hidden_size
        self.tied = bool(tied)
        self.tied_to = tied_to
        self.weight = None

    def param_specs(self):
        return [ParamSpec(self.prefix + "weight", (self.V, self.E), optional=self.tied)]

    def bind(self, params, ops):
        own = params.get(self.prefix + "weight")
        self.weight = own if own is not None else params[self.tied_to]

    def forward(self, ops, h, out_logits):
        with ops.section("head"):
            ops.gemm(h, self.weight, out_logits)
