"""RMSNorm fused with the residual sum.

``x * rsqrt(mean(x^2) + eps) * w`` with the statistics in float32; the reference places it before the mixer,
before the feed-forward and after the last block (models/src/llama.rs:401-408, 416-421, 474, 487).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import Begun, Norm, WeightedSum, WeightSpec, register_norm


class RMSNorm(Norm):
    def __init__(self, width: int, eps: float, name: str = "weight", offset: float = 0.0, scalar: bool = False):
        # ``name``: the tensor's name below the part's prefix ("weight" as checkpoints of the Llama family have it)
        # ``offset``: what is added to the stored tensor to make the weight (1 for weights stored around zero); such
        # a weight is kept in float32, since 1 + w has more digits than the checkpoint's dtype
        # ``scalar``: the checkpoint holds one number for all columns (a tensor without dimensions, or of one entry)
        self.width, self.eps, self.name, self.offset = int(width), float(eps), str(name), float(offset)
        self.scalar = bool(scalar)
        self.weight: Optional[torch.Tensor] = None
        self.weight_f32: Optional[torch.Tensor] = None
        self.act_dtype = torch.float32

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec(() if self.scalar else (self.width,), "norm" if self.offset == 0.0 else "norm_zero")}

    def load(self, get, device, act_dtype) -> None:
        self.weight = get(self.name).to(device).contiguous()
        if self.scalar:      # the kernels take a weight per column: the one number, as often as there are columns
            self.weight = self.weight.reshape(1).expand(self.width).contiguous()
        if self.offset != 0.0:
            self.weight = (self.weight.to(torch.float32) + self.offset).contiguous()
        self.weight_f32 = self.weight.to(torch.float32)
        self.act_dtype = act_dtype

    def device_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def add_norm(self, resid, delta, rows=None):
        if isinstance(delta, WeightedSum):
            # sublayers that ran side by side: their outputs are summed into the stream by the norm's own kernel
            if rows is None:
                return ops.add_normed(resid, delta.terms, None, 0.0, self.weight_f32, self.eps, self.act_dtype)
            # (rows are asked for behind the last block only: the stream takes the sum, then the rows are normed)
            ops.add_normed(resid, delta.terms, None, 0.0)
            delta = None
        return ops.add_rmsnorm(resid, delta, self.weight, self.eps, self.act_dtype, rows)

    def add_normed(self, resid, delta, next_norm=None, average=None):
        """``resid += self(delta)`` (in place): this norm stands behind a sublayer, whose output ``delta`` (a tensor,
        float32 planes or a ``WeightedSum`` of up to two such) it norms before the sum.  With ``next_norm`` (an
        RMSNorm) the same kernel also returns ``next_norm(resid)`` in the activation dtype.  ``average`` = (results
        float32 [blocks + 1, T, W], n, weights float32 [n]): the new rows are kept as results[n - 1] and the stream
        becomes ``sum_(j < n) weights[j] results[j]`` before ``next_norm`` reads it."""
        terms = delta.terms if isinstance(delta, WeightedSum) else [(delta, 1.0)]
        if average is not None:
            results, n, weights = average
            if next_norm is None:
                return ops.depth_average(resid, terms, self.weight_f32, self.eps, results, n, weights)
            return ops.depth_average(resid, terms, self.weight_f32, self.eps, results, n, weights,
                                     next_norm.weight_f32, next_norm.eps, next_norm.act_dtype)
        if next_norm is None:
            return ops.add_normed(resid, terms, self.weight_f32, self.eps)
        return ops.add_normed(resid, terms, self.weight_f32, self.eps, next_norm.weight_f32, next_norm.eps,
                              next_norm.act_dtype)

    # the norm begun by its neighbours (bfloat16 steps of at most 16 rows): see kernels/gemm_bf16.py; with many rows
    # the library adds its product to the residual rows itself, and the norm reads them once
    def add_product(self, resid, x, w, tiled=None):
        if self.act_dtype is not torch.bfloat16 or w.dtype is not torch.bfloat16:
            return None
        from ..kernels import gemm_bf16
        from .linear import Normed, as_tensor
        y = gemm_bf16.try_linear_resid(x, w, resid, self.weight, self.eps, tiled)
        if y is not None:
            y.norm = self
            return y
        if gemm_bf16.try_addmm_resid(as_tensor(x), w, resid):
            return Normed(self.add_norm(resid, None), self)
        return None

    def embed(self, table, tokens):
        if self.act_dtype is not torch.bfloat16 or tokens.numel() > 16 or table.shape[1] != self.width:
            return None
        resid, u, ss = ops.embed_begin_norm(tokens, table, self.weight)
        return resid, Begun(u, ss, self.eps, self.width, self)


register_norm("rmsnorm", RMSNorm)
