"""A residual stream kept in several copies (hyper-connections), and the embedding and final norm that go with it.

The stream of a step is float32 [S, T, W]: S copies x_1 .. x_S of every row, all equal to the embedding's output at
the start.  A sublayer q of a ``StreamBlock`` has three small tensors, ``in`` [S], ``mix`` [S, S] (indexed [from, to])
and ``out`` [S]:

    u = sum_s in[s] x_s;   y = sublayer(norm(u));   x_t <- sum_s mix[s, t] x_s + out[t] y   (all copies at once).

The update of one sublayer and the read of the next are one kernel (``ops.stream_step``), so a block hands the block
behind it its last sublayer's output together with the weights of its update, still to be applied (``StreamUpdate``),
as the other blocks hand on a pending delta.  What leaves the model is the norm of the sum of the copies
(``StreamsNorm``).  With ``copies=None`` a block has no such tensors and one copy: u = x, x <- x + y, the plain
pre-norm residual.

``BigramEmbedding``: ``table[token] * scale`` plus a row of a second table chosen by the token and the one before it,
``(prev * mul_prev + token * mul_cur) mod buckets``, the table's last row (number ``buckets``) for a request's first
token.  The token before an entry's first is per-request state: one int32, kept like a mixer's state.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Block, FeedForward, Mixer, Norm, Part, StateSpec, WeightedSum, WeightSpec, register_block, register_norm
from .block import _join


@dataclasses.dataclass
class StreamUpdate:
    """A sublayer's output ``y`` ([T, W] or float32 planes) with the weights that mix it into the stream's copies."""
    y: torch.Tensor
    mix: torch.Tensor
    out: torch.Tensor


class StreamWeights(Part):
    """``in``, ``mix`` and ``out`` of one sublayer, kept in float32; or, without tensors, those of a single copy."""

    def __init__(self, copies: Optional[int], prefix: str):
        self.copies, self.prefix = copies, str(prefix)
        self.w_in = self.mix = self.out = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        if self.copies is None:
            return {}
        s = self.copies
        # (a checkpoint of one copy may come without them: they are then one, the plain residual)
        opt = s == 1
        return {f"{self.prefix}.in": WeightSpec((s,), "linear", mean=1.0 / s, std=0.1, optional=opt),
                f"{self.prefix}.out": WeightSpec((s,), "linear", mean=1.0, std=0.2, optional=opt),
                f"{self.prefix}.mix": WeightSpec((s, s), "near_identity", std=0.1, optional=opt)}

    def load(self, get, device, act_dtype) -> None:
        f32 = dict(device=device, dtype=torch.float32)
        if self.copies is None:
            self.w_in = self.mix = self.out = torch.ones(1, **f32)
            return
        def take(name, shape):
            try:
                return get(f"{self.prefix}.{name}").to(**f32).contiguous()
            except KeyError:
                if self.copies != 1:
                    raise
                return torch.ones(shape, **f32)
        self.w_in, self.mix, self.out = take("in", (1,)), take("mix", (1, 1)), take("out", (1,))


class StreamBlock(Block):
    """Pre-norm sublayers (mixer, then an optional feed-forward) around a stream of ``copies`` copies.

    ``names``: the children's prefixes below the layer's, in the order (norm1, norm2, mixer, feed-forward); the
    connection weights are ``hc1.*`` and ``hc2.*``.  A mixer with two normed branches may hand back a ``WeightedSum``:
    it is not supported here, the mixer's output is one tensor or float32 planes."""

    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Optional[Norm] = None,
                 feed_forward: Optional[FeedForward] = None, copies: Optional[int] = None,
                 names=("", "", "mix", "mlp"), connection_names=("hc1", "hc2")):
        if (norm2 is None) != (feed_forward is None):
            raise ValueError("the feed-forward and its norm come together or not at all")
        if copies is not None and not 1 <= copies <= ops.MAX_STREAM_COPIES:
            raise ValueError(f"1 to {ops.MAX_STREAM_COPIES} copies of the stream are supported, not {copies}")
        self.norm1, self.norm2, self.mixer, self.feed_forward = norm1, norm2, mixer, feed_forward
        self.copies, self.names = copies, tuple(names)
        self.hc1 = StreamWeights(copies, connection_names[0])
        self.hc2 = StreamWeights(copies, connection_names[1]) if feed_forward is not None else None

    @property
    def stream_copies(self) -> int:
        return self.copies or 1

    def _children(self):
        parts = (self.norm1, self.norm2, self.mixer, self.feed_forward)
        kids = [(n, p) for n, p in zip(self.names, parts) if p is not None]
        return kids + [("", self.hc1)] + ([("", self.hc2)] if self.hc2 is not None else [])

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {_join(n, k): ws for n, part in self._children() for k, ws in part.weight_specs().items()}

    def load(self, get, device, act_dtype) -> None:
        self.act_dtype = act_dtype
        for n, part in self._children():
            part.load(lambda rel, _n=n: get(_join(_n, rel)), device, act_dtype)

    def graph_safe(self) -> bool:
        return all(part.graph_safe() for _, part in self._children())

    def device_bytes(self) -> int:
        return sum(part.device_bytes() for _, part in self._children())

    @staticmethod
    def _read(norm):
        return norm.weight_f32, norm.eps

    def forward(self, resid, delta, ctx, cache):
        if resid.dim() != 3 or resid.shape[0] != self.stream_copies:
            raise RuntimeError(f"a block of {self.stream_copies} copies met a stream of shape {tuple(resid.shape)}")
        if delta is not None and not isinstance(delta, StreamUpdate):
            raise RuntimeError("a stream of copies takes the update of the block before it, nothing else")
        update = None if delta is None else (delta.y, delta.mix, delta.out)
        x = ops.stream_step(resid, update, (self.hc1.w_in, *self._read(self.norm1)), out_dtype=self.act_dtype)
        a = self.mixer.forward(x, ctx, cache)
        if isinstance(a, WeightedSum):
            raise RuntimeError("the mixer of a stream block hands back one tensor")
        if self.feed_forward is None:
            return StreamUpdate(a, self.hc1.mix, self.hc1.out)
        x = ops.stream_step(resid, (a, self.hc1.mix, self.hc1.out), (self.hc2.w_in, *self._read(self.norm2)),
                            out_dtype=self.act_dtype)
        return StreamUpdate(self.feed_forward.forward(x, ctx), self.hc2.mix, self.hc2.out)


class StreamsNorm(Norm):
    """The norm behind the last block of a stream of copies: the pending update is applied, the copies are summed and
    the sum is normed, at the wanted rows only."""

    def __init__(self, norm: Norm, copies: int):
        self.norm, self.copies = norm, int(copies)
        self.ones: Optional[torch.Tensor] = None

    def graph_safe(self) -> bool:
        return self.norm.graph_safe()

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return self.norm.weight_specs()

    def load(self, get, device, act_dtype) -> None:
        self.norm.load(get, device, act_dtype)
        self.ones = torch.ones(self.copies, dtype=torch.float32, device=device)

    def device_bytes(self) -> int:
        return self.norm.device_bytes()

    def add_norm(self, resid, delta, rows=None):
        if delta is not None and not isinstance(delta, StreamUpdate):
            raise RuntimeError("a stream of copies takes the update of the block before it, nothing else")
        update = None if delta is None else (delta.y, delta.mix, delta.out)
        return ops.stream_step(resid, update, (self.ones, self.norm.weight_f32, self.norm.eps), rows=rows,
                               out_dtype=self.norm.act_dtype)


class BigramEmbedding(Part):
    """See the module's text.  ``pairs`` = (buckets, mul_prev, mul_cur) or None for no second table; ``copies``: how
    many copies of the stream to write.  Tensors: ``name`` [vocab, width]; ``pair_name`` [buckets + 1, width]."""
    reads_context = True

    def __init__(self, vocab_size: int, width: int, scale: float = 1.0, pairs=None, copies: int = 1,
                 name: str = "embed", pair_name: str = "bigram"):
        self.vocab_size, self.width, self.scale, self.copies = int(vocab_size), int(width), float(scale), int(copies)
        self.pairs = None if pairs is None else tuple(int(v) for v in pairs)
        if self.pairs is not None and self.pairs[0] <= 0:
            raise ValueError("the table of pairs needs at least one bucket")
        self.name, self.pair_name = str(name), str(pair_name)
        self.weight: Optional[torch.Tensor] = None
        self.pair_table: Optional[torch.Tensor] = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = {self.name: WeightSpec((self.vocab_size, self.width), "embedding")}
        if self.pairs is not None:
            specs[self.pair_name] = WeightSpec((self.pairs[0] + 1, self.width), "embedding")
        return specs

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((1,), "int32") if self.pairs is not None else None

    def load(self, get, device, act_dtype) -> None:
        self.weight = get(self.name).to(device).contiguous()
        if self.pairs is not None:
            self.pair_table = get(self.pair_name).to(device=device, dtype=self.weight.dtype).contiguous()

    def device_bytes(self) -> int:
        return 0      # a step reads only the rows of its tokens

    def forward_step(self, ctx, cache) -> torch.Tensor:
        """The stream float32 [copies, T, W] of the step's tokens; ``cache.state`` holds the requests' last tokens."""
        buckets, mul_prev, mul_cur = self.pairs if self.pairs is not None else (0, 0, 0)
        return ops.bigram_embed(ctx.tokens, ctx.positions, ctx.token_seq, ctx.q_start, ctx.state_slots,
                                cache.state if self.pairs is not None else None, self.weight, self.pair_table, buckets,
                                mul_prev, mul_cur, self.scale, self.copies)


register_block("stream", StreamBlock)
register_norm("streams", StreamsNorm)
