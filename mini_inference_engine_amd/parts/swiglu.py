"""Dense gated feed-forward: down( act(gate(x)) * up(x) ), act = silu (z sigmoid(z)) unless the
constructor names another of kernels.api.ACTIVATIONS; gate and up fused as the rows of one matrix,
gate first (inference_engine/model.py:109-110,180-181).  ``tensor_names``: how the checkpoint calls
the three matrices after the prefix."""
from __future__ import annotations

from .base import FeedForward, ParamSpec, register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    lazy_input = True

    def __init__(self, width: int, intermediate: int, prefix: str, activation: str = "silu",
                 tensor_names=("gate_proj.weight", "up_proj.weight", "down_proj.weight"), float32_output: bool = False):
        from ..kernels.api import ACTIVATIONS
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation {activation!r}: one of {ACTIVATIONS}")
        self.width = int(width)
        self.intermediate = int(intermediate)
        self.prefix = prefix
        self.activation = activation
        self.tensor_names = tuple(tensor_names)
        self.float32_output = bool(float32_output)      # where the caller norms the output itself: hand it the 32-bit sums
        self.w_gate_up = None
        self.w_down = None

    def params(self):
        p, w, i = self.prefix, self.width, self.intermediate
        gate, up, down = self.tensor_names
        return [ParamSpec.stacked("w_gate_up", [(f"{p}.{gate}", (i, w)), (f"{p}.{up}", (i, w))]),
                ParamSpec.single("w_down", f"{p}.{down}", (w, i))]

    def forward(self, x, step, add_to=None):
        if self.activation == "silu":
            a = self.ops.linear_silu_mul(x, self.w_gate_up, self.intermediate)
        else:
            a = self.ops.linear_act_mul(x, self.w_gate_up, self.intermediate, self.activation)
        if self.float32_output and add_to is None:
            import torch
            return self.ops.linear(a, self.w_down, out_dtype=torch.float32)
        return self.ops.linear(a, self.w_down, add_to=add_to)
