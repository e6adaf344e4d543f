"""Delta-rule recurrence with a decay per key channel and a removal gate (a generalised delta rule).

Per head a state S [dim, dim] (key channel i, value channel j), zero before a request's first token:
    S <- diag(decay) S - (a * u) (u^T S) + k v^T      (both terms read the old S),     o = S^T r
with r, k, v = W h per head; u = k / sqrt(sum(k^2) + 1e-6) the head's unit key;
decay = exp(-decay_scale * sigmoid(W_w2 tanh(W_w1 h) + w0)) and a = sigmoid(W_a h + a_b) per head and key channel.
Each head's o is divided by its root mean square, the heads are concatenated, multiplied by a weight and by
sigmoid(W_g h), and go through the output projection.  Decay, gates, unit keys, state and the whole recurrence are
32-bit; the state lives in the request's state slot, which the cache zeroes when it hands the slot out, so a portion
that starts anywhere goes on from what the slot holds.

One product computes everything that reads h (r, k, v, g, a and the decay's inner activations); one kernel does the rest.
"""
from __future__ import annotations

import math

from .base import FixedState, Mixer, ParamSpec, register_mixer

DEFAULT_NAMES = dict(r="r", k="k", v="v", g="g", a="a", a_bias="a.b", w1="w1", w2="w2", w0="w0", norm="norm", o="o")


@register_mixer("delta_rule")
class DeltaRule(Mixer):
    def __init__(self, width: int, num_heads: int, dim: int, rank: int, eps: float, prefix: str,
                 decay_scale: float = math.exp(-0.5), float32_output: bool = False, tensor_names=None):
        self.width, self.num_heads, self.dim, self.rank = int(width), int(num_heads), int(dim), int(rank)
        if self.dim > 256:
            raise ValueError(f"states of {dim} x {dim} a head are beyond the 256 the recurrence kernel takes")
        self.eps, self.decay_scale, self.prefix = float(eps), float(decay_scale), prefix
        self.float32_output = bool(float32_output)
        self.names = dict(DEFAULT_NAMES, **(tensor_names or {}))
        n = self.num_heads * self.dim
        self.cols = dict(r=0, k=n, v=2 * n, g=3 * n, a=4 * n, w=5 * n)

    def params(self):
        nm, w, n = self.names, self.width, self.num_heads * self.dim
        name = lambda k: f"{self.prefix}.{nm[k]}"        # noqa: E731
        return [ParamSpec.stacked("w_in", [(name(k), (n, w)) for k in ("r", "k", "v", "g", "a")] + [(name("w1"), (self.rank, w))]),
                ParamSpec.single("w_decay", name("w2"), (n, self.rank)),
                ParamSpec.single("decay_bias", name("w0"), (n,)),
                ParamSpec.single("removal_bias", name("a_bias"), (n,)),
                ParamSpec.single("norm", name("norm"), (n,), init="scale"),
                ParamSpec.single("w_o", name("o"), (w, n))]

    def cache_requirement(self):
        return FixedState((self.num_heads, self.dim, self.dim), "float32")

    def prepare(self, device, dtype):
        import torch
        if getattr(self, "_prepared", False):
            return
        self._prepared = True
        rows = self.w_in.shape[0]
        if rows % 16:
            padded = torch.zeros((-(-rows // 16) * 16, self.width), dtype=self.w_in.dtype, device=self.w_in.device)
            padded[:rows] = self.w_in
            self.w_in = padded
        # everything inside the recurrence is 32-bit whatever the checkpoint stores
        for attr in ("w_decay", "decay_bias", "removal_bias", "norm"):
            setattr(self, attr, getattr(self, attr).float().contiguous())

    def forward(self, x, step, cache, add_to=None, sums=None, base=0):
        """``sums``: the float32 sums of a product that holds this part's ``w_in`` rows from column ``base`` on (a
        caller that stacked several parts' input matrices); ``x`` is then not read."""
        import torch
        ops = self.ops
        if sums is None:
            sums, base = ops.linear(x, self.w_in, out_dtype=torch.float32), 0
        cols = self.cols if base == 0 else {k: v + base for k, v in self.cols.items()}
        out = ops.delta_rule(sums, cols, self.num_heads, self.dim, self.w_decay, self.decay_bias, self.decay_scale,
                             self.removal_bias, self.norm, self.eps, cache.state, step)
        if add_to is None and self.float32_output:
            return ops.linear(out, self.w_o, out_dtype=torch.float32)
        return ops.linear(out, self.w_o, add_to=add_to)
