"""Configuration of the Vezodra decoder, read from its own ``config.json`` keys.

The file lists the layers one by one: each names its mixer kind (``attention``: softmax attention with a sink,
a temperature per head and a gate per head, whose values are its keys; or ``parallel``: sliding-window attention
beside a delta-rule recurrence), the mixer's sizes and constants and its feed-forward (``dense`` or none).
``loop`` names a stretch of layers that runs several times in a row with the same weights, ``canon`` the short
convolution on what every mixer reads.  Every size and constant that may differ between two models of the
design is a field here.  One size is in no key of the file, the inner size of the decay's two-matrix product:
it is read from the shape of the checkpoint's tensor (``reads_tensor_shapes``), or from the key ``rank`` that
this reader's own ``to_dict`` writes beside the other sizes.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, ModelConfig, _take_float, _take_int
from .zifelorn_config import DenseFFSpec, _section


@dataclass(frozen=True)
class RotaryAnglesSpec:
    """Pair i of the first ``dims`` numbers of a head turns by position * base^(-2i / dims) / factor."""
    base: float
    dims: int
    factor: float = 1.0

    @classmethod
    def from_dict(cls, d, where, head_dim):
        scaling = d.get("scaling")
        factor = 1.0 if scaling is None else _take_float(_section(d, "scaling", where), "factor")
        spec = cls(_take_float(d, "base"), _take_int(d, "dims", minimum=2), factor)
        if spec.dims % 2 or spec.dims > head_dim:
            raise ConfigError(f"config.json: {where}rot.dims {spec.dims} must be even and at most the head size {head_dim}")
        if not spec.base > 0 or not spec.factor > 0:
            raise ConfigError(f"config.json: {where}rot.base and rot.scaling.factor must be positive")
        return spec

    def to_dict(self):
        d = dict(base=self.base, dims=self.dims)
        if self.factor != 1.0:
            d["scaling"] = dict(factor=self.factor)
        return d


def _heads(d, where):
    heads, kv_heads = _take_int(d, "heads"), _take_int(d, "kv_heads")
    if heads % kv_heads:
        raise ConfigError(f"config.json: {where}heads {heads} is not a multiple of kv_heads {kv_heads}")
    return heads, kv_heads


@dataclass(frozen=True)
class SinkAttentionSpec:
    """Softmax attention over all earlier keys with one more term, of score 0 and no value, in every softmax's
    denominator; the values are the keys as projected; one temperature and one output gate a query head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotaryAnglesSpec
    kind = "attention"

    @classmethod
    def from_dict(cls, d, where, shapes=None):
        heads, kv_heads = _heads(d, where)
        dim = _take_int(d, "dim")
        spec = cls(heads, kv_heads, dim, _take_int(d, "vdim", default=dim), _take_float(d, "scale"),
                   RotaryAnglesSpec.from_dict(_section(d, "rot", where), where, dim))
        if spec.vdim != spec.dim:
            raise ConfigError(f"config.json: {where}vdim {spec.vdim} differs from dim {spec.dim}, but this mixer's values are its keys")
        return spec

    def to_dict(self):
        return dict(heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim, scale=self.scale, rot=self.rot.to_dict())


@dataclass(frozen=True)
class WindowAttentionSpec:
    """Softmax attention over the last ``window`` keys (None: all), queries and keys normed over their whole projection."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotaryAnglesSpec
    window: int | None

    @classmethod
    def from_dict(cls, d, where):
        heads, kv_heads = _heads(d, where)
        dim = _take_int(d, "dim")
        mask = d.get("mask")
        window = None if mask is None else _take_int(_section(d, "mask", where), "size")
        return cls(heads, kv_heads, dim, _take_int(d, "vdim", default=dim), _take_float(d, "scale"),
                   RotaryAnglesSpec.from_dict(_section(d, "rot", where), where, dim), window)

    def to_dict(self):
        d = dict(heads=self.heads, kv_heads=self.kv_heads, dim=self.dim, vdim=self.vdim, scale=self.scale, rot=self.rot.to_dict())
        if self.window is not None:
            d["mask"] = dict(size=self.window)
        return d


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Delta-rule recurrence: ``heads`` states of dim x dim; ``rank`` is the inner size of the decay's product."""
    heads: int
    dim: int
    rank: int

    def to_dict(self):
        return dict(heads=self.heads, dim=self.dim, rank=self.rank)


@dataclass(frozen=True)
class ParallelSpec:
    left: WindowAttentionSpec
    right: DeltaRuleSpec
    kind = "parallel"

    @classmethod
    def from_dict(cls, d, where, shapes=None, layer=0):
        right = _section(d, "right", where)
        rank = right.get("rank")
        name = f"l{layer}.mix.right.w1"
        if rank is None and shapes is not None and name in shapes:
            rank = int(shapes[name][0])
        if rank is None:
            raise ConfigError(f"config.json: {where}right.rank is not given and no checkpoint tensor {name} to read it from")
        if isinstance(rank, bool) or not isinstance(rank, int) or rank < 1:
            raise ConfigError(f"config.json: {where}right.rank must be a positive integer, found {rank!r}")
        return cls(WindowAttentionSpec.from_dict(_section(d, "left", where), where + "left."),
                   DeltaRuleSpec(_take_int(right, "heads"), _take_int(right, "dim"), rank))

    def to_dict(self):
        return dict(left=self.left.to_dict(), right=self.right.to_dict())


@dataclass(frozen=True)
class LoopSpec:
    """Layers start .. stop - 1 run ``times`` times in a row with the same weights; every pass has its own cache."""
    start: int
    stop: int
    times: int

    def to_dict(self):
        return dict(start=self.start, stop=self.stop, times=self.times)


@dataclass(frozen=True)
class VezodraLayer:
    mixer: Any
    mlp: Any

    def to_dict(self):
        return dict(type=self.mixer.kind, mixer=self.mixer.to_dict(), mlp=None if self.mlp is None else self.mlp.to_dict())


@dataclass(frozen=True)
class VezodraConfig(ModelConfig):
    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    canon_taps: int | None = None       # taps of the convolution on what a mixer reads; None: there is none
    loop: LoopSpec | None = None

    architecture = "Vezodra"
    reads_tensor_shapes = True          # from_dict takes the checkpoint's tensor shapes beside the dictionary

    def __post_init__(self):
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        if not self.norm_eps > 0:
            raise ConfigError(f"config.json: norm.eps must be positive, found {self.norm_eps}")
        if self.loop is not None:
            lp = self.loop
            if not 0 <= lp.start < lp.stop <= len(self.layers) or lp.times < 1:
                raise ConfigError(f"config.json: loop {lp.to_dict()} does not name a stretch of the {len(self.layers)} layers")

    def run_order(self) -> list[int]:
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        lp = self.loop
        return list(range(lp.start)) + list(range(lp.start, lp.stop)) * lp.times + list(range(lp.stop, n))

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], tensor_shapes=None) -> "VezodraConfig":
        raw = d.get("layers")
        if not isinstance(raw, (list, tuple)):
            raise ConfigError("config.json: 'layers' must be a list")
        layers = []
        for i, entry in enumerate(raw):
            where = f"layers[{i}]."
            if not isinstance(entry, Mapping):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
            kind = entry.get("type")
            mixer = _section(entry, "mixer", where)
            if kind == "attention":
                m = SinkAttentionSpec.from_dict(mixer, where + "mixer.")
            elif kind == "parallel":
                m = ParallelSpec.from_dict(mixer, where + "mixer.", tensor_shapes, i)
            else:
                raise ConfigError(f"config.json: {where}type {kind!r} is not computed here (attention, parallel)")
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}mlp must be null or of kind 'dense'")
                mlp = DenseFFSpec(_take_int(mlp, "ff"))
            layers.append(VezodraLayer(m, mlp))
        canon = d.get("canon")
        taps = None if canon is None else _take_int(_section(d, "canon", ""), "taps")
        loop = d.get("loop")
        if loop is not None:
            lp = _section(d, "loop", "")
            loop = LoopSpec(_take_int(lp, "start", minimum=0), _take_int(lp, "stop"), _take_int(lp, "times"))
        return cls(vocab=_take_int(d, "vocab"), width=_take_int(d, "width"), layers=tuple(layers),
                   norm_eps=_take_float(_section(d, "norm", ""), "eps"), canon_taps=taps, loop=loop)

    def to_dict(self) -> dict:
        d = dict(architecture=self.architecture, vocab=self.vocab, width=self.width, norm=dict(eps=self.norm_eps),
                 layers=[layer.to_dict() for layer in self.layers])
        if self.canon_taps is not None:
            d["canon"] = dict(taps=self.canon_taps)
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        return d
