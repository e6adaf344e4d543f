"""Two mixers that read the same input, joined after a norm each:
y = scale * (rmsnorm(left(h)) * w_left + rmsnorm(right(h)) * w_right), norms over the model width in 32-bit.
Each side keeps its own cache or state (CombinedCache members ``left`` and ``right``)."""
from __future__ import annotations

from .base import CombinedCache, Mixer, ParamSpec, register_mixer


@register_mixer("side_by_side")
class SideBySide(Mixer):
    def __init__(self, width: int, left: Mixer, right: Mixer, eps: float, left_norm_name: str, right_norm_name: str,
                 scale: float = 0.5):
        self.width, self.left, self.right, self.eps, self.scale = int(width), left, right, float(eps), float(scale)
        self.norm_names = (left_norm_name, right_norm_name)

    def children(self):
        return [self.left, self.right]

    def params(self):
        return [ParamSpec.single("left_norm", self.norm_names[0], (self.width,), init="scale"),
                ParamSpec.single("right_norm", self.norm_names[1], (self.width,), init="scale")]

    def cache_requirement(self):
        return CombinedCache([("left", self.left.cache_requirement()), ("right", self.right.cache_requirement())])

    def prepare(self, device, dtype):
        import torch
        self.left_norm, self.right_norm = self.left_norm.float().contiguous(), self.right_norm.float().contiguous()
        # Both sides read the same input: where each has one input matrix (``w_in``) and takes a product's sums, the
        # two matrices are stacked and one product serves both.
        self.w_in = None
        for side in (self.left, self.right):
            side.prepare(device, dtype)
        wl, wr = getattr(self.left, "w_in", None), getattr(self.right, "w_in", None)
        if wl is not None and wr is not None and wl.dtype == wr.dtype and wl.shape[1] == wr.shape[1]:
            self.w_in = torch.cat([wl, wr]).contiguous()
            self.right_base = wl.shape[0]
            self.left.w_in = self.w_in[:wl.shape[0]]
            self.right.w_in = self.w_in[wl.shape[0]:]

    def forward(self, x, step, cache, add_to=None):
        import torch
        ops = self.ops
        if self.w_in is not None:
            sums = ops.linear(x, self.w_in, out_dtype=torch.float32)
            yl = self.left.forward(None, step, cache.sub("left"), sums=sums, base=0)
            yr = self.right.forward(None, step, cache.sub("right"), sums=sums, base=self.right_base)
        else:
            yl = self.left.forward(x, step, cache.sub("left"))
            yr = self.right.forward(x, step, cache.sub("right"))
        stream = getattr(add_to, "stream", add_to)
        if stream is None:
            stream = torch.zeros((yl.shape[0], self.width), dtype=torch.float32, device=yl.device)
        ops.normed_sum_add(stream, [yl, yr], [self.left_norm, self.right_norm], self.eps, self.scale)
        return None if add_to is not None else stream
