"""The Rakuvik decoder put together from parts.

Every layer is a sandwich block (a norm before and behind each sublayer, every norm with ONE number for all columns)
whose result is kept: what the next layer, or the output, reads is a weighted sum of the embedding's rows and the
results of all layers so far (``l<i>.dwa``).  The mixer is, layer by layer, differential attention (two softmax
maps a head over one set of values; a layer may read an earlier layer's keys and values, ``kv_from``) or a minGRU
recurrence; the feed-forward a dense gated one with the tanh form of GELU, or routed experts (softmax scores, a
correction that only chooses, squared-ReLU experts weighed on their outputs, a gated expert that every token uses).
Tensor names are the checkpoint's own: ``embed``, ``l<i>.norm1`` / ``norm1b`` / ``norm2`` / ``norm2b``,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.dwa``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.rakuvik import DenseFeedForward, DifferentialMixer, ExpertsFeedForward, MinGruMixer, RakuvikConfig
from ..config.registry import register_architecture
from ..parts.base import make_part
from ..parts.block import DepthAverage
from ..parts.embedding import OutputHead, TokenEmbedding
from .spec import LayerCall, ModelSpec


def _mixer(m, width: int, eps: float):
    if isinstance(m, DifferentialMixer):
        rot = m.rot if m.rot is not None and m.rot.dims > 0 else None
        return make_part("mixer", "differential_attention", width=width, num_heads=m.heads, num_kv_heads=m.kv_heads,
                         head_size=m.dim, value_size=m.vdim, scale=m.scale, diff=m.diff, norm_eps=eps,
                         rotary_base=rot.base if rot else 10000.0, rotary_dim=rot.dims if rot else 0,
                         rotary_factor=rot.scaling.factor if rot and rot.scaling else 1.0,
                         owns_cache=m.kv_from is None)
    if isinstance(m, MinGruMixer):
        return make_part("mixer", "mingru", width=width, inner=m.width)
    raise TypeError(f"no part for mixer {m!r}")


def _feed_forward(f, width: int):
    if f is None:
        return None
    if isinstance(f, DenseFeedForward):
        return make_part("feed_forward", "swiglu", width=width, intermediate=f.ff, names=("gate", "up", "down"),
                         activation="gelu_tanh")
    if isinstance(f, ExpertsFeedForward):
        return make_part("feed_forward", "routed_experts", width=width, intermediate=f.expert.ff,
                         experts=f.router.experts, top=f.router.top, score="softmax", scale=f.router.scale,
                         correction=True, expert="relu2", shared=f.shared.ff if f.shared is not None else 0)
    raise TypeError(f"no part for feed-forward {f!r}")


def build_rakuvik(cfg: RakuvikConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps
    norm = lambda name: make_part("norm", "rmsnorm", width=w, eps=eps, name=name, scalar=True)
    layers, order = [], []
    for i, layer in enumerate(cfg.layers):
        ffn = _feed_forward(layer.mlp, w)
        norms = (norm("norm1"), norm("norm1b"), norm("norm2") if ffn else None, norm("norm2b") if ffn else None)
        layers.append((f"l{i}", make_part("block", "sandwich", norms=norms, mixer=_mixer(layer.mixer, w, eps),
                                          feed_forward=ffn, depth_average=DepthAverage(i + 2, "dwa"))))
        order.append(LayerCall(i, getattr(layer.mixer, "kv_from", None)))
    # a layer without a feed-forward may still carry the two norms of one in its checkpoint
    ignorable = tuple(rf"l{i}\.norm2b?" for i, layer in enumerate(cfg.layers) if layer.mlp is None)
    return ModelSpec(width=w, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
                     embedding=("", TokenEmbedding(cfg.vocab, w, name="embed")), layers=layers,
                     final_norm=("", norm("final.norm")), head=("", OutputHead(w, cfg.vocab, name="head")),
                     run_order=order, ignorable=ignorable)


for _name in RakuvikConfig.architectures:
    register_architecture(_name, RakuvikConfig, build_rakuvik, replace=True)
