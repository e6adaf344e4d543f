"""Vezodra: a decoder whose layers are listed one by one in its configuration, a stretch of them run several
times in a row with the same weights.

A layer adds mixer and feed-forward to the stream side by side, each behind a norm of its own of the same stream;
what the mixer reads first goes through a short causal convolution that is added to it.  Mixers: softmax attention
over all earlier keys with a sink, a temperature and an output gate per head and the keys as values (``attention``),
or sliding-window attention with normed queries and keys beside a delta-rule recurrence, joined after a norm
each (``parallel``).  The feed-forward is the dense gated one (SiLU) or absent.  The head is the embedding table.
Everything here is construction: sizes and constants come from VezodraConfig only.  Tensor names: ``embed``,
``final.norm``, ``l<i>.norm1|norm2``, ``l<i>.canon1``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.vezodra_config import ParallelSpec, SinkAttentionSpec, VezodraConfig
from ..parts import (DecoderSpec, DeltaRule, Embedding, LayerCall, LMHead, ParallelBlock, ResidualConv, RMSNorm,
                     RotaryHalfAngles, RotaryInterleaved, SideBySide, SoftmaxAttention, SwiGLU)


def build_vezodra(cfg: VezodraConfig) -> DecoderSpec:
    w, eps = cfg.width, cfg.norm_eps
    rotations = {}          # one position-encoding part for each distinct (kind, dims, base, factor)

    def rotation(kind, rot):
        key = (kind, rot.dims, rot.base, rot.factor)
        if key not in rotations:
            rotations[key] = kind(rot.dims, rot.base, rot.factor)
        return rotations[key]

    layers = []
    for i, layer in enumerate(cfg.layers):
        m, f, p = layer.mixer, layer.mlp, f"l{i}"
        if isinstance(m, SinkAttentionSpec):
            mixer = SoftmaxAttention(w, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, rotation(RotaryInterleaved, m.rot),
                                     prefix=f"{p}.mix", sink=0.0, values_from_keys=True, head_temperature=True,
                                     head_gate=True, eps=eps)
        elif isinstance(m, ParallelSpec):
            a, d = m.left, m.right
            left = SoftmaxAttention(w, a.heads, a.kv_heads, a.dim, a.vdim, a.scale, rotation(RotaryHalfAngles, a.rot),
                                    prefix=f"{p}.mix.left", window=a.window, qk_norm=True, eps=eps, float32_output=True)
            right = DeltaRule(w, d.heads, d.dim, d.rank, eps, prefix=f"{p}.mix.right", float32_output=True)
            mixer = SideBySide(w, left, right, eps, f"{p}.mix.left.out", f"{p}.mix.right.out", scale=0.5)
        else:
            raise TypeError(f"layer {i}: no part for mixer {m!r}")
        ff = norm2 = None
        if f is not None:
            norm2 = RMSNorm(w, eps, f"{p}.norm2")
            ff = SwiGLU(w, f.ff, prefix=f"{p}.mlp", tensor_names=("gate", "up", "down"))
        conv = None if cfg.canon_taps is None else ResidualConv(w, cfg.canon_taps, f"{p}.canon1")
        layers.append(ParallelBlock(RMSNorm(w, eps, f"{p}.norm1"), mixer, norm2, ff, input_conv=conv))
    embedding = Embedding(cfg.vocab, w, "embed")
    return DecoderSpec(embedding=embedding, layers=layers, final_norm=RMSNorm(w, eps, "final.norm"),
                       head=LMHead(cfg.vocab, w, "embed", tied_to=embedding),
                       schedule=[LayerCall(i) for i in cfg.run_order()], stop_token_ids=(), max_position=None,
                       vocab_size=cfg.vocab)


def _shape(vocab, width, ff, heads, kv_heads, dim, window, rec_heads, rec_dim, rank, sink_heads, sink_kv_heads, sink_dim,
           repeats, times):
    """A named size: ``repeats`` times the run (parallel, attention, parallel), the middle layer of the first run
    looped ``times`` times."""
    rot = dict(base=10000.0, dims=dim, scaling=dict(factor=2.0))
    par = dict(left=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, mask=dict(size=window), rot=rot),
               right=dict(heads=rec_heads, dim=rec_dim, rank=rank))
    att = dict(heads=sink_heads, kv_heads=sink_kv_heads, dim=sink_dim, vdim=sink_dim, scale=sink_dim ** -0.5,
               rot=dict(base=10000.0, dims=sink_dim // 2))
    dense = dict(kind="dense", ff=ff)
    layers = []
    for _ in range(repeats):
        layers += [dict(type="parallel", mixer=par, mlp=dense), dict(type="attention", mixer=att, mlp=dense),
                   dict(type="parallel", mixer=par, mlp=dense)]
    return dict(vocab=vocab, width=width, norm=dict(eps=1e-6), canon=dict(taps=4), loop=dict(start=1, stop=2, times=times),
                layers=layers)


SHAPES = {
    "vezodra-tiny": _shape(vocab=320, width=64, ff=112, heads=4, kv_heads=2, dim=16, window=24, rec_heads=2, rec_dim=16, rank=8,
                           sink_heads=3, sink_kv_heads=1, sink_dim=32, repeats=1, times=2),
    "vezodra-1b": _shape(vocab=32000, width=2048, ff=5632, heads=32, kv_heads=4, dim=64, window=1024, rec_heads=16, rec_dim=64,
                         rank=64, sink_heads=16, sink_kv_heads=4, sink_dim=128, repeats=6, times=1),
}

register_architecture("Vezodra", VezodraConfig, build_vezodra, shapes=SHAPES, replace=True)
