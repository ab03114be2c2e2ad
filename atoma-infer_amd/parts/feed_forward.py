"""Dense gated feed-forward: ``down(act(gate(x)) * up(x))``, no biases; act is SiLU (SwiGLU:
models/src/llama.rs:362-366, 372-374) or, for designs that ask for it, the tanh form of GELU.

gate and up are fused into one [2 I, width] matrix at load time, so one product feeds the SiLU-multiply kernel.
When I is a multiple of 16 the rows are interleaved in blocks of 16 (16 gate rows, then the 16 up rows of the
same outputs): a lane of the weight-streaming MFMA product then holds a gate value and its up value, and the
activation runs in that product's epilogue for few rows of x.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import FeedForward, WeightSpec, register_feed_forward
from .linear import linear, linear_delta


class SwiGLU(FeedForward):
    def __init__(self, width: int, intermediate: int,
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight"), activation: str = "silu"):
        # ``names``: the tensors of the gate, up and down matrices below the part's prefix
        # ``activation``: of the gate, "silu" or "gelu_tanh" (0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))))
        if activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not supported (known: {', '.join(ops.GATE_ACTIVATIONS)})")
        self.activation = str(activation)
        self.width, self.inter, self.names = int(width), int(intermediate), tuple(names)
        self.block = 0
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_gate_up_tiled = self.w_down_tiled = None
        self.w_down: Optional[torch.Tensor] = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.names[0]: WeightSpec((self.inter, self.width)),
                self.names[1]: WeightSpec((self.inter, self.width)),
                self.names[2]: WeightSpec((self.width, self.inter))}

    def load(self, get, device, act_dtype) -> None:
        g, u = get(self.names[0]), get(self.names[1])
        dt = g.dtype if g.dtype is u.dtype else torch.float32
        g, u = g.to(device=device, dtype=dt), u.to(device=device, dtype=dt)
        self.block = 16 if self.inter % 16 == 0 else 0
        if self.block:
            gu = torch.stack([g.view(self.inter // 16, 16, self.width), u.view(self.inter // 16, 16, self.width)], dim=1)
            self.w_gate_up = gu.reshape(2 * self.inter, self.width).contiguous()
        else:
            self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = get(self.names[2]).to(device).contiguous()
        # second copies of the matrices in the order the streaming kernels' waves read them, for steps of few rows
        self.w_gate_up_tiled = self.w_down_tiled = None
        if act_dtype is torch.bfloat16 and self.w_gate_up.dtype is torch.bfloat16 and self.w_down.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            plan = gemm_bf16.tiled_plan(2 * self.inter, self.width, swiglu=True) if self.block else None
            if plan is not None:
                self.w_gate_up_tiled = gemm_bf16.tile_weight(self.w_gate_up, *plan)
            self.w_down_tiled = gemm_bf16.tile_copies_resid(self.w_down)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_gate_up, self.w_down))

    accepts_begun = True
    takes_sink = True

    def forward(self, x, ctx, sink=None):
        h = None
        if self.block and x.dtype is torch.bfloat16 and self.w_gate_up.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            h = gemm_bf16.try_linear_swiglu(x, self.w_gate_up, self.w_gate_up_tiled, self.activation)
        if h is None:
            h = ops.swiglu(linear(x, self.w_gate_up), block=self.block, act=self.activation)
        return linear_delta(h, self.w_down, sink, self.w_down_tiled)


class DenseFeedForward(FeedForward):
    """A feed-forward without a gate: ``down(act(up(x)))``, no biases; ``activation`` "relu2" is the square of relu."""

    def __init__(self, width: int, intermediate: int, names=("up", "down"), activation: str = "relu2"):
        if activation != "relu2":
            raise ValueError(f"activation {activation!r} is not supported (known: relu2)")
        self.width, self.inter, self.names, self.activation = int(width), int(intermediate), tuple(names), activation
        self.w_up = self.w_down = self.w_up_tiled = self.w_down_tiled = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        return {self.names[0]: WeightSpec((self.inter, self.width)), self.names[1]: WeightSpec((self.width, self.inter))}

    def load(self, get, device, act_dtype) -> None:
        self.w_up = get(self.names[0]).to(device).contiguous()
        self.w_down = get(self.names[1]).to(device).contiguous()
        self.w_up_tiled = self.w_down_tiled = None
        if act_dtype is torch.bfloat16 and self.w_up.dtype is torch.bfloat16 and self.w_down.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            plan = gemm_bf16.tiled_plan(self.inter, self.width, swiglu=False)
            if plan is not None:
                self.w_up_tiled = gemm_bf16.tile_weight(self.w_up, *plan)
            self.w_down_tiled = gemm_bf16.tile_copies_resid(self.w_down)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_up, self.w_down))

    def forward(self, x, ctx, sink=None):
        u = linear(x, self.w_up, tiled=self.w_up_tiled)
        return linear_delta(ops.dense_act(u, x.dtype, self.activation), self.w_down, sink, self.w_down_tiled)


register_feed_forward("swiglu", SwiGLU)
register_feed_forward("dense", DenseFeedForward)
