"""The Bafilorn decoder put together from parts.

The embedding is a scaled table plus a row of a second table chosen by the token and the one before it.  The residual
stream is kept in ``streams`` copies that every sublayer reads as a weighted sum and updates through a small mixing
matrix (``stream`` blocks); every layer is pre-norm (weights stored around zero) with a mixer and, where the layer has
one, a dense feed-forward whose activation is the square of relu.  The mixer is, layer by layer, attention over a
cached latent with a rotated key part (``latent_attention``), linear attention with a decay per head (``lightning``),
or two mixers side by side whose normed outputs are averaged (``parallel``: attention in chunks whose values are its
keys, and a gated linear recurrence).  A run of layers may be gone through several times with the same weights, each
pass with caches and states of its own (``loop``).  Tensor names are the checkpoint's own: ``embed``, ``bigram``,
``l<i>.norm1``, ``l<i>.hc1.in`` / ``mix`` / ``out``, ``l<i>.mix.*``, ``l<i>.mlp.up`` / ``down``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.bafilorn import BafilornConfig, LatentMixer, LightningMixer, ParallelMixerConfig
from ..config.registry import register_architecture
from ..parts.base import make_part
from ..parts.embedding import OutputHead
from ..parts.streams import BigramEmbedding, StreamsNorm
from .spec import LayerCall, ModelSpec


def _mixer(m, width: int, eps: float):
    if isinstance(m, LatentMixer):
        rot = m.rot
        return make_part("mixer", "rotary_latent_attention", width=width, num_heads=m.heads, head_size=m.dim,
                         rotary_size=m.rot_dim, value_size=m.vdim, rank=m.kv_rank, q_rank=m.q_rank, scale=m.scale,
                         norm_eps=eps, rotary_base=rot.base if rot is not None else 10000.0,
                         rotary_dim=rot.dims if rot is not None else 0)
    if isinstance(m, LightningMixer):
        return make_part("mixer", "lightning_attention", width=width, heads=m.heads, dim=m.dim, vdim=m.vdim,
                         decay=m.decay, norm_eps=eps)
    if isinstance(m, ParallelMixerConfig):
        l, r = m.left, m.right
        rot = l.rot
        scaling = rot.scaling.to_dict() if rot is not None and rot.scaling is not None else None
        left = make_part("mixer", "gated_tied_value_attention", width=width, num_heads=l.heads,
                         num_kv_heads=l.kv_heads, head_size=l.dim, scale=l.scale,
                         rotary_base=rot.base if rot is not None else 10000.0,
                         rotary_dim=rot.dims if rot is not None else 0, rotary_scaling=scaling, interleaved=False,
                         chunk=l.mask.size if l.mask is not None else None, unit_sink=True, bias=True)
        right = make_part("mixer", "gated_linear_recurrence", width=width, inner=r.width, blocks=r.blocks, taps=r.conv)
        norms = [make_part("norm", "rmsnorm", width=width, eps=eps, name="out") for _ in range(2)]
        return make_part("mixer", "parallel", branches=[left, right], scales=[0.5, 0.5], names=["left", "right"],
                         out_norms=norms)
    raise TypeError(f"no part for mixer {m!r}")


def build_bafilorn(cfg: BafilornConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps
    norm = lambda name: make_part("norm", "rmsnorm", width=w, eps=eps, name=name, offset=1.0)
    layers = []
    for i, layer in enumerate(cfg.layers):
        ffn = norm2 = None
        if layer.mlp is not None:
            ffn = make_part("feed_forward", "dense", width=w, intermediate=layer.mlp.ff, names=("up", "down"))
            norm2 = norm("norm2")
        layers.append((f"l{i}", make_part("block", "stream", norm1=norm("norm1"), mixer=_mixer(layer.mixer, w, eps),
                                          norm2=norm2, feed_forward=ffn, copies=cfg.streams)))
    n = len(layers)
    order = [LayerCall(i) for i in range(n)]
    if cfg.loop is not None:
        lo, hi = cfg.loop.start, cfg.loop.stop
        order = [LayerCall(i) for i in range(lo)]
        for _ in range(cfg.loop.times):
            order += [LayerCall(i) for i in range(lo, hi)]
        order += [LayerCall(i) for i in range(hi, n)]
    copies = cfg.streams or 1
    bg = cfg.embedding.bigram
    embedding = BigramEmbedding(cfg.vocab, w, scale=cfg.embedding.scale,
                                pairs=(bg.buckets, bg.mul_prev, bg.mul_cur) if bg is not None else None, copies=copies,
                                name="embed", pair_name="bigram")
    return ModelSpec(width=w, vocab_size=cfg.vocab, max_positions=cfg.max_positions, embedding=("", embedding),
                     layers=layers, final_norm=("", StreamsNorm(norm("final.norm"), copies)),
                     head=("", OutputHead(w, cfg.vocab, name="head")), run_order=order)


for _name in BafilornConfig.architectures:
    register_architecture(_name, BafilornConfig, build_bafilorn, replace=True)
