"""Dense gated feed-forward: down( silu(gate(x)) * up(x) ), silu(z) = z sigmoid(z),
gate and up fused as the rows of one matrix, gate first
(inference_engine/model.py:109-110,180-181)."""
from __future__ import annotations

from .base import FeedForward, ParamSpec, register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    lazy_input = True

    def __init__(self, width: int, intermediate: int, prefix: str):
        self.width = int(width)
        self.intermediate = int(intermediate)
        self.prefix = prefix
        self.w_gate_up = None
        self.w_down = None

    def params(self):
        p, w, i = self.prefix, self.width, self.intermediate
        return [ParamSpec.stacked("w_gate_up", [(f"{p}.gate_proj.weight", (i, w)), (f"{p}.up_proj.weight", (i, w))]),
                ParamSpec.single("w_down", f"{p}.down_proj.weight", (w, i))]

    def forward(self, x, step, add_to=None):
        a = self.ops.linear_silu_mul(x, self.w_gate_up, self.intermediate)
        return self.ops.linear(a, self.w_down, add_to=add_to)
