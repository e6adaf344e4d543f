"""Zifelorn: a decoder whose layers are listed one by one in its configuration.

A layer is a mixer (attention through a cached latent, or a gated linear recurrence) and an optional
feed-forward (dense and gated, or routed experts), each followed by an RMSNorm on its output before it is
added to the stream; the branches read the stream itself.  The embedding is scaled, the head is the embedding
table (unscaled) times a logit scale.  A latent-attention layer may read the latent cache of an earlier
layer instead of making its own.  Everything here is construction: sizes and constants come from
ZifelornConfig only.  Tensor names: ``embed``, ``final.norm``, ``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zifelorn_config import DenseFFSpec, LatentAttentionSpec, MoEFFSpec, RglruSpec, ZifelornConfig
from ..parts import (RGLRU, BranchNormBlock, DecoderSpec, Embedding, LatentAttention, LayerCall, LMHead, RMSNorm,
                     RotaryInterleaved, RoutedExperts, SwiGLU)


def build_zifelorn(cfg: ZifelornConfig) -> DecoderSpec:
    w, eps = cfg.width, cfg.norm_eps
    rotations = {}          # one position-encoding part for each distinct (dims, base)
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        m, f, p = layer.mixer, layer.mlp, f"l{i}"
        cache_of = None
        if isinstance(m, LatentAttentionSpec):
            rot = rotations.setdefault((m.rot.dims, m.rot.base), RotaryInterleaved(m.rot.dims, m.rot.base))
            mixer = LatentAttention(w, m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.q_rank, m.scale, eps, rot,
                                    prefix=f"{p}.mix", has_kv=m.kv_from is None)
            cache_of = m.kv_from            # every layer runs once, so run-order entry j is layer j
        elif isinstance(m, RglruSpec):
            mixer = RGLRU(w, m.width, m.blocks, m.conv, prefix=f"{p}.mix")
        else:
            raise TypeError(f"layer {i}: no part for mixer {m!r}")
        if f is None:
            ff = norm2 = None
        else:
            norm2 = RMSNorm(w, eps, f"{p}.norm2")
            if isinstance(f, DenseFFSpec):
                ff = SwiGLU(w, f.ff, prefix=f"{p}.mlp", activation="gelu_tanh", tensor_names=("gate", "up", "down"),
                            float32_output=True)
            elif isinstance(f, MoEFFSpec):
                ff = RoutedExperts(w, f.expert_ff, f.experts, f.top, prefix=f"{p}.mlp", activation="relu2")
            else:
                raise TypeError(f"layer {i}: no part for feed-forward {f!r}")
        layers.append(BranchNormBlock(mixer, RMSNorm(w, eps, f"{p}.norm1"), ff, norm2))
        schedule.append(LayerCall(i, cache_of=cache_of))
    embedding = Embedding(cfg.vocab, w, "embed", scale=cfg.embedding_scale)
    return DecoderSpec(embedding=embedding, layers=layers, final_norm=RMSNorm(w, eps, "final.norm"),
                       head=LMHead(cfg.vocab, w, "embed", tied_to=embedding, scale=cfg.logit_scale), schedule=schedule,
                       stop_token_ids=(), max_position=None, vocab_size=cfg.vocab)


def _layer(kind, mixer, mlp):
    return dict(type=kind, mixer=mixer, mlp=mlp)


def _shape(vocab, width, heads, dim, rot_dim, vdim, kv_rank, q_rank, channels, blocks, ff, experts, top, expert_ff, repeats):
    """A named size: ``repeats`` times the run (latent attention + dense, latent attention + experts, recurrence +
    dense, latent attention reading the second layer's latent + experts)."""
    att = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank,
               scale=(dim + rot_dim) ** -0.5, rot=dict(base=10000.0, dims=rot_dim))
    rec = dict(width=channels, blocks=blocks, conv=4)
    dense = dict(kind="dense", ff=ff)
    moe = dict(kind="moe", expert=dict(ff=expert_ff), router=dict(experts=experts, top=top))
    layers = []
    for r in range(repeats):
        base = 4 * r
        layers += [_layer("latent_attention", att, dense), _layer("latent_attention", att, moe),
                   _layer("rglru", rec, dense), _layer("latent_attention", dict(att, kv_from=base + 1), moe)]
    return dict(vocab=vocab, width=width, embedding=dict(scale=float(width) ** 0.5), norm=dict(eps=1e-6),
                logit_scale=1.0, layers=layers)


# Named sizes: one for tests and the command line's examples, one with the widths of a 1B-class model.
SHAPES = {
    "zifelorn-tiny": _shape(vocab=320, width=64, heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=48, channels=96,
                            blocks=3, ff=112, experts=5, top=2, expert_ff=48, repeats=1),
    "zifelorn-1b": _shape(vocab=32000, width=2048, heads=16, dim=128, rot_dim=64, vdim=128, kv_rank=192, q_rank=768,
                          channels=2560, blocks=10, ff=5632, experts=16, top=2, expert_ff=1408, repeats=5),
}

register_architecture("Zifelorn", ZifelornConfig, build_zifelorn, shapes=SHAPES, replace=True)
