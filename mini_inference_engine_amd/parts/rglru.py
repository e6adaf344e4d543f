"""Recurrent mixer with a real-gated linear recurrent unit (the recurrent block of Griffin: De et al.,
"Griffin: Mixing Gated Linear Recurrences with Local Attention for Efficient Language Models").

Two branches of ``channels`` each: y = gelu_tanh(W_y x + b_y) and u = conv(W_x x + b_x), a causal convolution
per channel over the last ``taps`` inputs (zeros before a request's start, no activation).  With u cut into
``blocks`` equal parts, r = sigmoid(A_b u_b + a_b) and i = sigmoid(I_b u_b + i_b) (square matrices per part);
a = exp(-decay_scale * r * softplus(lam)); S_t = a S_{t-1} + sqrt(1 - a^2) * i * u, S = 0 before the first
token; the mixer returns W_o (S * y).  Gates, decay, state and everything else inside the recurrence are 32-bit.

Per request the part keeps S [channels] and the last taps - 1 inputs of the convolution, both float32, in the
request's state slot; the cache zeroes a slot when it hands it out, so a portion that starts anywhere simply
goes on from what the slot holds.
"""
from __future__ import annotations

from dataclasses import dataclass

from .base import CacheRequirement, Mixer, ParamSpec, register_mixer

DEFAULT_NAMES = dict(y="y", y_bias="y.b", x="x", x_bias="x.b", conv="conv", conv_bias="conv.b", a_gate="ra",
                     a_gate_bias="ra.b", i_gate="ri", i_gate_bias="ri.b", lam="lam", o="o")


@dataclass(frozen=True)
class RecurrentState(CacheRequirement):
    """Per request: the recurrence's state [channels] and the convolution's last inputs [taps - 1, channels]."""
    channels: int
    taps: int

    def allocate(self, num_pages, page_size, num_slots, device, act_dtype):
        import torch
        return {"state": torch.zeros((num_slots, self.channels), dtype=torch.float32, device=device),
                "tail": torch.zeros((num_slots, max(1, self.taps - 1), self.channels), dtype=torch.float32, device=device)}

    def reset_slot(self, tensors, slot):
        tensors["state"][slot].zero_()
        tensors["tail"][slot].zero_()


@register_mixer("rglru")
class RGLRU(Mixer):
    def __init__(self, width: int, channels: int, blocks: int, taps: int, prefix: str, decay_scale: float = 8.0,
                 tensor_names=None):
        self.width, self.channels, self.blocks, self.taps = int(width), int(channels), int(blocks), int(taps)
        if self.channels % self.blocks:
            raise ValueError(f"{channels} channels do not split into {blocks} equal parts")
        if self.taps < 1:
            raise ValueError("the convolution needs at least one tap")
        self.decay_scale = float(decay_scale)
        self.prefix = prefix
        self.names = dict(DEFAULT_NAMES, **(tensor_names or {}))

    def params(self):
        n, w, C, B = self.names, self.width, self.channels, self.blocks
        name = lambda k: f"{self.prefix}.{n[k]}"        # noqa: E731
        bw = C // B
        return [ParamSpec.stacked("w_in", [(name("y"), (C, w)), (name("x"), (C, w))]),
                ParamSpec.stacked("b_in", [(name("y_bias"), (C,)), (name("x_bias"), (C,))]),
                ParamSpec.single("conv", name("conv"), (C, self.taps)),
                ParamSpec.single("conv_bias", name("conv_bias"), (C,), init="zeros"),
                ParamSpec.stacked("w_gates", [(name("a_gate"), (B, bw, bw)), (name("i_gate"), (B, bw, bw))]),
                ParamSpec.stacked("b_gates", [(name("a_gate_bias"), (B, bw)), (name("i_gate_bias"), (B, bw))]),
                ParamSpec.single("lam", name("lam"), (C,)),
                ParamSpec.single("w_o", name("o"), (w, C))]

    def cache_requirement(self):
        return RecurrentState(self.channels, self.taps)

    def prepare(self, device, dtype):
        # the recurrence, its gates' biases and the convolution are 32-bit whatever the checkpoint stores
        for attr in ("b_in", "conv", "conv_bias", "b_gates", "lam"):
            setattr(self, attr, getattr(self, attr).float().contiguous())

    def forward(self, x, step, cache, add_to=None):
        import torch
        ops, C = self.ops, self.channels
        state, tail = cache.tensors["state"], cache.tensors["tail"]
        sums = ops.linear(x, self.w_in, out_dtype=torch.float32)          # [T, y | x] before their biases
        b_y, b_x = self.b_in[:C], self.b_in[C:]
        u = ops.causal_conv(sums, C, C, b_x, self.conv, self.conv_bias, tail, step)
        gates = ops.grouped_linear(u, self.w_gates, self.b_gates, x_groups=self.blocks)
        out = ops.rglru_scan(u, gates, self.lam, sums, 0, b_y, sums, C, b_x, state, tail, step, self.taps, self.decay_scale)
        return ops.linear(out, self.w_o, out_dtype=torch.float32)
