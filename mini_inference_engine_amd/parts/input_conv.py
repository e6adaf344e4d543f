"""A short causal convolution added to what a mixer reads: c(h)[t] = h[t] + sum_j w[:, j] * h[t - (K - 1) + j], per
channel, zeros before a request's first token, no bias.  The last K - 1 inputs of a request are part of its state
(ConvTail, in its state slot), so a portion that starts anywhere continues the convolution."""
from __future__ import annotations

from dataclasses import dataclass

from .base import CacheRequirement, ParamSpec, Part


@dataclass(frozen=True)
class ConvTail(CacheRequirement):
    """Per request: the convolution's last taps - 1 inputs [taps - 1, channels], float32, oldest first."""
    channels: int
    taps: int

    def allocate(self, num_pages, page_size, num_slots, device, act_dtype):
        import torch
        return {"tail": torch.zeros((num_slots, max(1, self.taps - 1), self.channels), dtype=torch.float32, device=device)}

    def reset_slot(self, tensors, slot):
        tensors["tail"][slot].zero_()


class ResidualConv(Part):
    def __init__(self, channels: int, taps: int, weight_name: str):
        if taps < 1:
            raise ValueError("the convolution needs at least one tap")
        self.channels, self.taps, self.weight_name = int(channels), int(taps), weight_name
        self.weight = None

    def params(self):
        return [ParamSpec.single("weight", self.weight_name, (self.channels, self.taps))]

    def cache_requirement(self):
        return ConvTail(self.channels, self.taps)

    def prepare(self, device, dtype):
        self.weight = self.weight.float().contiguous()

    def forward(self, h, step, cache, out_dtype=None):
        """h [T, channels] float32 -> h + conv(h) in the activation dtype; the request's tail moves on."""
        return self.ops.residual_conv(h, self.weight, cache.tensors["tail"], step, out_dtype=out_dtype)
