"""Configuration of the Zifelorn decoder, read from its own ``config.json`` keys.

The file lists the layers one by one: each names its mixer kind (``latent_attention`` or ``rglru``), the
mixer's sizes and constants, and its feed-forward (``dense``, ``moe`` or none).  Every size and every
constant that may differ between two models of the design is a field here; nothing about a particular
model is assumed (layer order, head counts, ranks, expert counts, whether two sizes happen to be equal).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .model_config import ConfigError, ModelConfig, _take_float, _take_int


def _section(d: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    v = d.get(key)
    if not isinstance(v, Mapping):
        raise ConfigError(f"config.json: {where}'{key}' must be an object")
    return v


@dataclass(frozen=True)
class RotarySpec:
    base: float
    dims: int


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention through a low-rank latent: per head ``dim`` unrotated and ``rot_dim`` rotated query/key dims,
    values of ``vdim``, keys and values expanded from a latent of ``kv_rank``, queries from one of ``q_rank``.
    ``kv_from``: the layer whose latent and rotated key part this layer reads instead of making its own."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: RotarySpec
    kv_from: int | None = None
    kind = "latent_attention"

    @classmethod
    def from_dict(cls, d, where):
        rot = _section(d, "rot", where)
        spec = cls(heads=_take_int(d, "heads"), dim=_take_int(d, "dim"), rot_dim=_take_int(d, "rot_dim"),
                   vdim=_take_int(d, "vdim"), kv_rank=_take_int(d, "kv_rank"), q_rank=_take_int(d, "q_rank"),
                   scale=_take_float(d, "scale"), rot=RotarySpec(_take_float(rot, "base"), _take_int(rot, "dims")),
                   kv_from=None if d.get("kv_from") is None else _take_int(d, "kv_from", minimum=0))
        if spec.rot.dims % 2 or spec.rot.dims > spec.rot_dim:
            raise ConfigError(f"config.json: {where}rot.dims {spec.rot.dims} must be even and at most rot_dim {spec.rot_dim}")
        if not spec.rot.base > 0:
            raise ConfigError(f"config.json: {where}rot.base must be positive")
        return spec

    def to_dict(self):
        d = dict(heads=self.heads, dim=self.dim, rot_dim=self.rot_dim, vdim=self.vdim, kv_rank=self.kv_rank,
                 q_rank=self.q_rank, scale=self.scale, rot=dict(base=self.rot.base, dims=self.rot.dims))
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class RglruSpec:
    """Recurrent block with a real-gated linear recurrent unit: two branches of ``width`` channels, a causal
    convolution of ``conv`` taps on one of them, gates that are block-diagonal in ``blocks`` equal parts."""
    width: int
    blocks: int
    conv: int
    kind = "rglru"

    @classmethod
    def from_dict(cls, d, where):
        spec = cls(width=_take_int(d, "width"), blocks=_take_int(d, "blocks"), conv=_take_int(d, "conv"))
        if spec.width % spec.blocks:
            raise ConfigError(f"config.json: {where}width {spec.width} is not a multiple of blocks {spec.blocks}")
        return spec

    def to_dict(self):
        return dict(width=self.width, blocks=self.blocks, conv=self.conv)


@dataclass(frozen=True)
class DenseFFSpec:
    ff: int
    kind = "dense"

    def to_dict(self):
        return dict(kind="dense", ff=self.ff)


@dataclass(frozen=True)
class MoEFFSpec:
    experts: int
    top: int
    expert_ff: int
    kind = "moe"

    def to_dict(self):
        return dict(kind="moe", expert=dict(ff=self.expert_ff), router=dict(experts=self.experts, top=self.top))


def _feed_forward(d, where):
    if d is None:
        return None
    if not isinstance(d, Mapping):
        raise ConfigError(f"config.json: {where}mlp must be an object or null")
    kind = d.get("kind")
    if kind == "dense":
        return DenseFFSpec(_take_int(d, "ff"))
    if kind == "moe":
        router = _section(d, "router", where)
        spec = MoEFFSpec(_take_int(router, "experts"), _take_int(router, "top"),
                         _take_int(_section(d, "expert", where), "ff"))
        if spec.top > spec.experts:
            raise ConfigError(f"config.json: {where}router.top {spec.top} exceeds router.experts {spec.experts}")
        return spec
    raise ConfigError(f"config.json: {where}mlp.kind {kind!r} is not computed here (dense, moe)")


_MIXERS = {"latent_attention": LatentAttentionSpec, "rglru": RglruSpec}


@dataclass(frozen=True)
class ZifelornLayer:
    mixer: Any
    mlp: Any

    def to_dict(self):
        return dict(type=self.mixer.kind, mixer=self.mixer.to_dict(), mlp=None if self.mlp is None else self.mlp.to_dict())


@dataclass(frozen=True)
class ZifelornConfig(ModelConfig):
    vocab: int
    width: int
    layers: tuple
    norm_eps: float
    embedding_scale: float
    logit_scale: float

    architecture = "Zifelorn"

    def __post_init__(self):
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        if not self.norm_eps > 0:
            raise ConfigError(f"config.json: norm.eps must be positive, found {self.norm_eps}")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if isinstance(m, LatentAttentionSpec) and m.kv_from is not None:
                j = m.kv_from
                src = self.layers[j].mixer if 0 <= j < i else None
                if not isinstance(src, LatentAttentionSpec) or src.kv_from is not None:
                    raise ConfigError(f"config.json: layers[{i}].mixer.kv_from = {j} must name an earlier "
                                      "latent_attention layer that makes its own latent")
                if (src.kv_rank, src.rot_dim, src.rot) != (m.kv_rank, m.rot_dim, m.rot):
                    raise ConfigError(f"config.json: layers[{i}] reads layer {j}'s latent; kv_rank, rot_dim and rot "
                                      "of the two must be equal")

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "ZifelornConfig":
        raw = d.get("layers")
        if not isinstance(raw, (list, tuple)):
            raise ConfigError("config.json: 'layers' must be a list")
        layers = []
        for i, entry in enumerate(raw):
            where = f"layers[{i}]."
            if not isinstance(entry, Mapping):
                raise ConfigError(f"config.json: layers[{i}] must be an object")
            kind = entry.get("type")
            if kind not in _MIXERS:
                raise ConfigError(f"config.json: {where}type {kind!r} is not computed here ({sorted(_MIXERS)})")
            layers.append(ZifelornLayer(_MIXERS[kind].from_dict(_section(entry, "mixer", where), where + "mixer."),
                                        _feed_forward(entry.get("mlp"), where)))
        return cls(vocab=_take_int(d, "vocab"), width=_take_int(d, "width"), layers=tuple(layers),
                   norm_eps=_take_float(_section(d, "norm", ""), "eps"),
                   embedding_scale=_take_float(_section(d, "embedding", ""), "scale"),
                   logit_scale=_take_float(d, "logit_scale"))

    def to_dict(self) -> dict:
        return dict(architecture=self.architecture, vocab=self.vocab, width=self.width,
                    embedding=dict(scale=self.embedding_scale), norm=dict(eps=self.norm_eps),
                    logit_scale=self.logit_scale, layers=[layer.to_dict() for layer in self.layers])
