"""Arrangements of parts around the residual stream.

``PreNormBlock``: ``h = x + mixer(norm1(x))``, ``y = h + ffn(norm2(h))`` (models/src/llama.rs:393-410).  The residual
stream is float32; each sum is fused with the norm that follows it, so a block receives the previous block's
output as a pending ``delta`` and returns its own.

``SideBySideBlock``: one norm whose output both sublayers read, ``h = norm1(x)``, ``y = x + (mixer(h) + ffn(h))``; the
two outputs travel on unsummed, and the kernel of the norm that reads the stream next adds them in.

``SandwichBlock``: a norm before and a norm behind each sublayer, ``h = x + norm1b(mixer(norm1(x)))``,
``y = h + norm2b(ffn(norm2(h)))``; the feed-forward half may be absent.  One kernel norms a sublayer's output, adds
it to the stream and applies the norm that reads the stream next.  With a ``DepthAverage`` the block's result y is
kept beside those of all blocks before it, and what the stream carries on is a weighted sum of them all.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Begun, Block, FeedForward, Mixer, Norm, Part, WeightSpec, register_block
from .linear import Normed, ResidualSink

BEGUN_ROWS = 16      # rows of a step up to which products begin and finish norms (kernels.gemm_bf16.BEGUN_MAX_M)


class PreNormBlock(Block):
    def __init__(self, norm1: Norm, mixer: Mixer, norm2: Norm, feed_forward: FeedForward,
                 names=("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")):
        self.norm1, self.mixer, self.norm2, self.feed_forward = norm1, mixer, norm2, feed_forward
        self.names = tuple(names)

    def _children(self):
        return zip(self.names, (self.norm1, self.mixer, self.norm2, self.feed_forward))

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {f"{n}.{k}": ws for n, part in self._children() for k, ws in part.weight_specs().items()}

    def load(self, get, device, act_dtype) -> None:
        for n, part in self._children():
            part.load(lambda rel, _n=n: get(f"{_n}.{rel}"), device, act_dtype)

    def graph_safe(self) -> bool:
        return all(part.graph_safe() for _, part in self._children())

    def device_bytes(self) -> int:
        return sum(part.device_bytes() for _, part in self._children())

    fuses_next_norm = True

    def entry_norm(self):
        return self.norm1

    @staticmethod
    def _normed(norm, resid, pending, reader):
        """The input of ``reader``: ``pending`` is either a delta still to be added and normed, or ``norm`` already
        begun or finished by the product that made it (which has also added it to ``resid``)."""
        if isinstance(pending, Normed):
            if pending.norm is not norm:
                raise RuntimeError("a finished norm reached another norm than the one it was made for")
            return pending.data
        if isinstance(pending, Begun):
            if pending.norm is not norm:
                raise RuntimeError("a begun norm reached another norm than the one it was begun for")
            return pending if reader.accepts_begun else pending.tensor()
        return norm.add_norm(resid, pending)

    def forward(self, resid, delta, ctx, cache, next_norm=None):
        x = self._normed(self.norm1, resid, delta, self.mixer)
        if self.mixer.takes_sink:
            a = self.mixer.forward(x, ctx, cache, sink=ResidualSink(resid, self.norm2))
        else:
            a = self.mixer.forward(x, ctx, cache)
        x = self._normed(self.norm2, resid, a, self.feed_forward)
        if self.feed_forward.takes_sink and next_norm is not None:
            return self.feed_forward.forward(x, ctx, sink=ResidualSink(resid, next_norm))
        return self.feed_forward.forward(x, ctx)


def _join(prefix: str, rel: str) -> str:
    return f"{prefix}.{rel}" if prefix and rel else prefix or rel


class DepthAverage(Part):
    """The weights of a block that hands on, instead of its own result, a weighted sum of the results of all blocks
    up to itself: with X_0 the embedding's rows and X_(j+1) the result of the block at run-order position j, the
    block at position i leaves ``sum_(j <= i + 1) w[j] X_j`` in the stream.  ``count`` = i + 2 weights, one tensor
    (``name``), kept and applied in float32."""

    def __init__(self, count: int, name: str = "dwa"):
        if count < 2:
            raise ValueError("a depth average has at least the embedding's rows and one block's result to weigh")
        self.count, self.name = int(count), str(name)
        self.weights: Optional[torch.Tensor] = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.count,), "tail_heavy", mean=0.3 / self.count, std=0.05)}

    def load(self, get, device, act_dtype) -> None:
        self.weights = get(self.name).to(device=device, dtype=torch.float32).contiguous()


class SandwichBlock(Block):
    """``norms`` = (before the mixer, behind it, before the feed-forward, behind it); the last two and the
    feed-forward are None for a layer that has the mixer only.  ``names``: the children's prefixes below the
    layer's, in the order (norms..., mixer, feed-forward, depth average); a part whose tensor carries its whole name
    has prefix "".  ``depth_average``: see ``DepthAverage``; the model then hands ``forward`` the results kept so far
    (``keeps_results``)."""

    def __init__(self, norms, mixer: Mixer, feed_forward: Optional[FeedForward] = None,
                 names=("", "", "", "", "mix", "mlp", ""), depth_average: Optional[DepthAverage] = None):
        self.norm1, self.norm1b, self.norm2, self.norm2b = norms
        self.mixer, self.feed_forward = mixer, feed_forward
        if (feed_forward is None) != (self.norm2 is None) or (feed_forward is None) != (self.norm2b is None):
            raise ValueError("the feed-forward and its two norms come together or not at all")
        self.names = tuple(names) + ("",) * (7 - len(names))
        self.depth_average = depth_average
        self.keeps_results = depth_average is not None

    def _children(self):
        parts = (self.norm1, self.norm1b, self.norm2, self.norm2b, self.mixer, self.feed_forward, self.depth_average)
        return [(n, p) for n, p in zip(self.names, parts) if p is not None]

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {_join(n, k): ws for n, part in self._children() for k, ws in part.weight_specs().items()}

    def load(self, get, device, act_dtype) -> None:
        for n, part in self._children():
            part.load(lambda rel, _n=n: get(_join(_n, rel)), device, act_dtype)

    def graph_safe(self) -> bool:
        return all(part.graph_safe() for _, part in self._children())

    def device_bytes(self) -> int:
        return sum(part.device_bytes() for _, part in self._children())

    fuses_next_norm = True

    def entry_norm(self):
        return self.norm1

    def forward(self, resid, delta, ctx, cache, next_norm=None, results=None, position=0):
        if isinstance(delta, Normed):
            if delta.norm is not self.norm1:
                raise RuntimeError("a finished norm reached another norm than the one it was made for")
            x = delta.data
        elif isinstance(delta, Begun):
            if delta.norm is not self.norm1:
                raise RuntimeError("a begun norm reached another norm than the one it was begun for")
            x = delta.tensor()
        else:
            x = self.norm1.add_norm(resid, delta)
        a = self.mixer.forward(x, ctx, cache)
        last, out = self.norm1b, a
        if self.feed_forward is not None:
            x = self.norm1b.add_normed(resid, a, self.norm2)
            last, out = self.norm2b, self.feed_forward.forward(x, ctx)
        if self.depth_average is None:
            x = last.add_normed(resid, out, next_norm)
        else:
            # the same kernel keeps the block's result and leaves the weighted sum of all results in the stream
            if results is None or position + 2 != self.depth_average.count:
                raise RuntimeError(f"a depth average of {self.depth_average.count} weights at run-order position "
                                   f"{position}: it weighs the embedding's rows and one result per block so far")
            x = last.add_normed(resid, out, next_norm, average=(results, position + 2, self.depth_average.weights))
        return Normed(x, next_norm) if next_norm is not None else None


class SideBySideBlock(Block):
    """``x += mixer(norm1(x)) + feed_forward(norm1(x))``: one norm, read by both sublayers; the feed-forward may be
    absent.  ``names``: the children's prefixes below the layer's, in the order (norm, mixer, feed-forward)."""

    def __init__(self, norm1: Norm, mixer: Mixer, feed_forward: Optional[FeedForward] = None,
                 names=("", "mix", "mlp")):
        self.norm1, self.mixer, self.feed_forward = norm1, mixer, feed_forward
        self.names = tuple(names)

    def _children(self):
        return [(n, p) for n, p in zip(self.names, (self.norm1, self.mixer, self.feed_forward)) if p is not None]

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {_join(n, k): ws for n, part in self._children() for k, ws in part.weight_specs().items()}

    def load(self, get, device, act_dtype) -> None:
        for n, part in self._children():
            part.load(lambda rel, _n=n: get(_join(_n, rel)), device, act_dtype)

    def graph_safe(self) -> bool:
        return all(part.graph_safe() for _, part in self._children())

    def device_bytes(self) -> int:
        return sum(part.device_bytes() for _, part in self._children())

    fuses_next_norm = True

    def entry_norm(self):
        return self.norm1

    def forward(self, resid, delta, ctx, cache, next_norm=None):
        from .base import WeightedSum
        if isinstance(delta, (Normed, Begun)):
            # the block before has added its outputs to the stream and begun or finished this block's norm
            if delta.norm is not self.norm1:
                raise RuntimeError("a begun or finished norm reached another norm than the one it was made for")
            x = delta.data if isinstance(delta, Normed) else delta
        else:
            x = self.norm1.add_norm(resid, delta)
        few = isinstance(x, Begun) or (x.dtype is torch.bfloat16 and x.shape[0] <= BEGUN_ROWS)

        def reads(part):
            return x if not isinstance(x, Begun) or part.accepts_begun else x.tensor()

        if self.feed_forward is None:
            if self.mixer.takes_sink and few and next_norm is not None:
                return self.mixer.forward(reads(self.mixer), ctx, cache, sink=ResidualSink(resid, next_norm))
            return self.mixer.forward(reads(self.mixer), ctx, cache)
        # Steps of few rows: both sublayers' last products add themselves to the stream's rows (the mixer's first, so
        # that the feed-forward's, which also begins the next norm, sees the rows complete), and no kernel of its own
        # sums them.  What the mixer's product begins of a norm is dropped: its rows lacked the feed-forward's share.
        if few and next_norm is not None and self.mixer.takes_sink and self.feed_forward.takes_sink:
            a = self.mixer.forward(reads(self.mixer), ctx, cache, sink=ResidualSink(resid, next_norm))
            if not isinstance(a, (Begun, Normed)):      # the product could not: its delta joins the stream here
                ops.add_normed(resid, a.terms if isinstance(a, WeightedSum) else [(a, 1.0)], None, 0.0)
            return self.feed_forward.forward(reads(self.feed_forward), ctx, sink=ResidualSink(resid, next_norm))
        a = self.mixer.forward(reads(self.mixer), ctx, cache)
        return WeightedSum([(a, 1.0), (self.feed_forward.forward(reads(self.feed_forward), ctx), 1.0)])


register_block("pre_norm", PreNormBlock)
register_block("side_by_side", SideBySideBlock)
register_block("sandwich", SandwichBlock)
