"""Feed-forward of routed experts: each token runs the ``top`` experts whose router logits are largest.

z = W_r x + b_r in 32-bit; the chosen experts' shares are the softmax over their logits alone; an expert is
W_down act(W_up x) without biases (act: the square of relu unless another of kernels.api.ACTIVATIONS is named);
the output is the share-weighted sum.  The experts' matrices are kept stacked, [experts, ff, width] and
[experts, width, ff], so that one grouped product serves all of them.
"""
from __future__ import annotations

from .base import FeedForward, ParamSpec, register_feed_forward


@register_feed_forward("routed_experts")
class RoutedExperts(FeedForward):
    def __init__(self, width: int, inner: int, num_experts: int, top: int, prefix: str, activation: str = "relu2",
                 router_bias: bool = True, tensor_names=None):
        from ..kernels.api import ACTIVATIONS
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation {activation!r}: one of {ACTIVATIONS}")
        if not 1 <= top <= num_experts:
            raise ValueError(f"top {top} of {num_experts} experts")
        self.width, self.inner, self.num_experts, self.top = int(width), int(inner), int(num_experts), int(top)
        self.prefix, self.activation, self.router_bias = prefix, activation, bool(router_bias)
        self.names = dict(dict(router="router", router_bias="router.b", expert="e{e}", up="up", down="down"),
                          **(tensor_names or {}))

    def params(self):
        n, p, w, f, E = self.names, self.prefix, self.width, self.inner, self.num_experts
        expert = lambda e, m: f"{p}.{n['expert'].format(e=e)}.{n[m]}"        # noqa: E731
        specs = [ParamSpec.single("w_router", f"{p}.{n['router']}", (E, w)),
                 ParamSpec.stacked("w_up", [(expert(e, "up"), (f, w)) for e in range(E)]),
                 ParamSpec.stacked("w_down", [(expert(e, "down"), (w, f)) for e in range(E)])]
        if self.router_bias:
            specs.append(ParamSpec.single("b_router", f"{p}.{n['router_bias']}", (E,), init="zeros"))
        return specs

    def prepare(self, device, dtype):
        if self.router_bias:
            self.b_router = self.b_router.float().contiguous()      # router logits are 32-bit

    def forward(self, x, step, add_to=None):
        import torch
        ops, E = self.ops, self.num_experts
        logits = ops.linear(x, self.w_router, out_dtype=torch.float32)
        experts, shares = ops.route_topk(logits, self.b_router if self.router_bias else None, self.top)
        return ops.routed_experts(x, experts, shares, self.w_up.view(E, self.inner, self.width),
                                  self.w_down.view(E, self.width, self.inner), self.activation)
