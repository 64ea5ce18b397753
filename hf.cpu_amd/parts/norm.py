"""Root-mean-square norm with a learned scale."""
from ..registry import register_part
from .base import ParamSpec, Part


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    """``y_i = x_i * (1 / sqrt(mean(x^2) + eps)) * w_i`` with the mean of squares in
    fp32 (src/mathx.c:65-75; the reference sums in fp64)."""
    graph_safe = True
    can_be_lazy = True          # forward(..., lazy=True) may leave the division to the products that read the output


    def __init__(self, size, eps, prefix=""):
        super().__init__(prefix)
        self.size = size
        self.eps = float(eps)
        self.weight = None

    def param_specs(self):
        return [ParamSpec(self.prefix + "weight", (self.size,), "vector", ("one_plus_normal", 0.1))]

    def bind(self, params, ops):
        self.weight = params[self.prefix + "weight"]

    def forward(self, ops, x, out, rows=None, lazy=False):
        """``out[r] = norm(x[rows[r]])`` (``rows`` None: every row in order). ``lazy``: the caller promises that
        ``out`` is read through ``ops.gemm`` alone (a part that says ``lazy_input_ok``); see ``Ops.rmsnorm``."""
        ops.rmsnorm(x, self.weight, self.eps, out, rows, lazy=lazy)
