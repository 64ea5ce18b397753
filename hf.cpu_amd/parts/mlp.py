"""Dense feed-forward parts."""
import torch

from .. import memory

from ..registry import register_part
from ..status import ENOTSUP, fail
from .base import ParamSpec, Part


@register_part("feed_forward", "gated_mlp")
class GatedMLP(Part):
    """``x += Wdown (act(Wgate h) * (Wup h))`` with ``act(g) = g / (1 + exp(-g))``
    (src/model.c:612-623, src/mathx.c:34). Gate and up share their input and are held
    as one matrix, gate rows first."""
    graph_safe = True
    lazy_input_ok = True


    def __init__(self, hidden_size, intermediate_size, activation="silu", prefix=""):
        super().__init__(prefix)
        if activation != "silu":
            fail(ENOTSUP, f"gated_mlp: activation '{activation}' is not implemented")
        self.E, self.F = hidden_size, intermediate_size
        self.w_gate_up = self.w_down = None
        self.fused = False

    def param_specs(self):
        p = self.prefix
        return [ParamSpec(p + "gate_proj.weight", (self.F, self.E)),
                ParamSpec(p + "up_proj.weight", (self.F, self.E)),
                ParamSpec(p + "down_proj.weight", (self.E, self.F))]

    def bind(self, params, ops):
        p = self.prefix
        g, u = params[p + "gate_proj.weight"], params[p + "up_proj.weight"]
        dt = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        # On the matrix cores gate and up rows are interleaved in blocks of 32, so that the product's
        # last step can form silu(gate) * up without storing gate and up.
        self.fused = ops.can_fuse_swiglu(g, u)
        if self.fused:
            memory.note(f"{p}gate and up, interleaved")
            self.w_gate_up = ops.interleave_gate_up(g, u)
        else:
            self.w_gate_up = memory.cat([g.to(dt), u.to(dt)], 0, f"{p}gate and up in one matrix")
        self.w_down = params[p + "down_proj.weight"]

    def forward(self, ops, step, h, x):
        T = h.shape[0]
        act = ops.scratch("ffn_act", (T, self.F), ops.act_dtype)
        if self.fused:
            with ops.section("gate_up"):           # the activation is the product's last step
                ops.gemm(h, self.w_gate_up, act, swiglu=True)
        else:
            gu = ops.scratch("gate_up", (T, 2 * self.F), ops.act_dtype)
            with ops.section("gate_up"):
                ops.gemm(h, self.w_gate_up, gu)
            with ops.section("silu"):
                ops.swiglu(gu, act)
        with ops.section("down"):
            ops.gemm(act, self.w_down, x, accumulate=True, defer=True)
