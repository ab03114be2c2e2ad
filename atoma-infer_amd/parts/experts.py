"""Feed-forward layers of many small experts, of which every token uses a few.

``RoutedExperts``: router logits ``z = W_r x`` in float32; scores ``s = sigmoid(z)`` or ``softmax(z)`` over all
experts; the ``top`` experts with the largest ``s + correction`` are chosen (``correction``: a tensor of one number
an expert that only chooses; none: the scores alone; the lower index wins a tie) and weighed by ``s * scale`` as
they are, without renormalising.  Two forms of expert, no biases:

* ``swiglu``: ``W_down (silu(W_gate z) * (W_up z))``; the weight multiplies the expert's *input*,
  ``out = sum_e expert_e(s_e x)``;
* ``relu2``: ``W_down relu(W_up z)^2``, no gate; the weight multiplies the expert's *output*,
  ``out = sum_e s_e expert_e(x)``.

``shared`` adds an expert of the same form and of ``shared`` columns that every token uses, multiplied by
``sigmoid(W_sg x)``, one number a token (``relu2`` experts).

The chosen (token, choice) pairs are ordered by expert on the device (no count or index passes the host, so a step
may be recorded into a graph), and two grouped products walk them tile by tile; the second writes choice c of
every token into plane c, and the norm behind the layer adds the planes in order.  In bfloat16 the products run on
the matrix cores (float32 sums): the inputs are gathered in the experts' order first, and the first product
applies the activation in its epilogue (an expert's gate and up rows are interleaved in blocks of 16 at load time
for silu(gate) * up).  The 32-bit path, and sizes that the matrix-core kernel does not take (a width that is no
multiple of 32, an expert width that is no multiple of 32), run true float32 multiply-adds.

Tensors: ``router`` [experts, width]; ``correction`` [experts]; ``e<i>.gate``, ``e<i>.up`` [ff, width],
``e<i>.down`` [width, ff]; ``shared.up`` [shared, width], ``shared.down`` [width, shared], ``shared.sg`` [1, width].
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import FeedForward, WeightedSum, WeightSpec, register_feed_forward
from .linear import linear, linear_delta


class RoutedExperts(FeedForward):
    def __init__(self, width: int, intermediate: int, experts: int, top: int, score: str = "sigmoid",
                 scale: float = 1.0, correction: bool = False, expert: str = "swiglu", shared: int = 0):
        if not 0 < top <= experts or experts > 1024:
            raise ValueError(f"{top} of {experts} experts: top must be at least 1 and at most the number of experts "
                             f"(up to 1,024)")
        if score not in ("sigmoid", "softmax") or expert not in ("swiglu", "relu2"):
            raise ValueError("scores are 'sigmoid' or 'softmax', experts 'swiglu' or 'relu2'")
        if shared and expert != "relu2":
            raise ValueError("a shared expert comes with 'relu2' experts")
        self.width, self.inter, self.experts, self.top = int(width), int(intermediate), int(experts), int(top)
        self.score, self.scale, self.has_correction = str(score), float(scale), bool(correction)
        self.expert, self.shared = str(expert), int(shared)
        self.gated = self.expert == "swiglu"
        self.w_router = self.w_gate_up = self.w_down = self.correction = None
        self.w_shared_up = self.w_shared_down = self.w_shared_down_tiled = None
        self.mfma = False       # set at load time: the products run on the matrix cores

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        specs = {"router": WeightSpec((self.experts, self.width), std=0.5)}
        if self.has_correction:
            specs["correction"] = WeightSpec((self.experts,), std=0.3)
        for e in range(self.experts):
            if self.gated:
                specs[f"e{e}.gate"] = WeightSpec((self.inter, self.width))
            specs[f"e{e}.up"] = WeightSpec((self.inter, self.width), std=0.02 if self.gated else 0.2)
            specs[f"e{e}.down"] = WeightSpec((self.width, self.inter))
        if self.shared:
            specs["shared.up"] = WeightSpec((self.shared, self.width), std=0.2)
            specs["shared.down"] = WeightSpec((self.width, self.shared))
            specs["shared.sg"] = WeightSpec((1, self.width), std=0.3)
        return specs

    def load(self, get, device, act_dtype) -> None:
        self.w_router = get("router").to(device).contiguous()
        self.correction = get("correction").to(device=device, dtype=torch.float32).contiguous() \
            if self.has_correction else None
        ups = [get(f"e{e}.up") for e in range(self.experts)]
        gates = [get(f"e{e}.gate") for e in range(self.experts)] if self.gated else []
        self.w_down = torch.stack([get(f"e{e}.down") for e in range(self.experts)]).to(device).contiguous()
        rows = (2 if self.gated else 1) * self.inter
        self.mfma = (act_dtype is torch.bfloat16 and self.w_down.dtype is torch.bfloat16
                     and all(t.dtype is torch.bfloat16 for t in gates + ups) and self.inter % 16 == 0
                     and ops.expert_gemm_mfma_ok(rows, self.width)
                     and ops.expert_gemm_mfma_ok(self.width, self.inter))
        if not self.gated:
            gu = ups
        elif self.mfma:
            # [experts, 2 ff, width]: blocks of 16 gate rows, each followed by the 16 up rows of the same outputs
            gu = [torch.stack([g.view(-1, 16, self.width), u.view(-1, 16, self.width)], dim=1).reshape(-1, self.width)
                  for g, u in zip(gates, ups)]
        else:
            gu = [torch.cat([g, u], dim=0) for g, u in zip(gates, ups)]     # gate rows, then up rows
        self.w_gate_up = torch.stack(gu).to(device).contiguous()
        if self.shared:
            # the shared expert's first matrix and the row of its gate are one product
            up, sg = get("shared.up"), get("shared.sg")
            dt = up.dtype if up.dtype is sg.dtype else torch.float32
            parts = [up.to(device=device, dtype=dt), sg.to(device=device, dtype=dt).view(1, self.width)]
            if (-(self.shared + 1)) % 64:      # whole tiles for the matrix-core products
                parts.append(torch.zeros(((-(self.shared + 1)) % 64, self.width), dtype=dt, device=device))
            self.w_shared_up = torch.cat(parts, dim=0).contiguous()
            self.w_shared_down = get("shared.down").to(device).contiguous()
            self.w_shared_down_tiled = None
            if act_dtype is torch.bfloat16 and self.w_shared_down.dtype is torch.bfloat16:
                from ..kernels import gemm_bf16
                self.w_shared_down_tiled = gemm_bf16.tile_copies_resid(self.w_shared_down)

    def device_bytes(self) -> int:
        """The router, the chosen share of the experts (what a step of one token reads) and the shared expert."""
        per_expert = (self.w_gate_up.numel() + self.w_down.numel()) // self.experts * self.w_down.element_size()
        shared = sum(w.numel() * w.element_size() for w in (self.w_shared_up, self.w_shared_down) if w is not None)
        return self.w_router.numel() * self.w_router.element_size() + self.top * per_expert + shared

    def _routed(self, x, ids, weights):
        t = x.shape[0]
        slots = t * self.top
        flat = weights.view(-1)
        # the weight goes into a gated expert's input and onto an ungated expert's output
        w_in, w_out = (flat, None) if self.gated else (None, flat)
        if self.mfma and x.dtype is torch.bfloat16:
            # tiles of 128 places where an expert has about a hundred or more (prompts): a weight fragment then
            # serves twice as many rows
            tile_m = 128 if slots >= 96 * self.experts else 64
            perm, offsets, tiles = ops.route_group(ids.view(-1), self.experts, tile_m)
            xs = ops.gather_scale(x, w_in, perm, self.top)
            h = torch.empty((slots, self.inter), dtype=torch.bfloat16, device=x.device)
            ops.expert_gemm_mfma(xs, self.w_gate_up, h, perm, offsets, tiles, self.top, swiglu=self.gated,
                                 relu2=not self.gated, tile_m=tile_m)
            out = torch.empty((self.top, t, self.width), dtype=torch.float32, device=x.device)
            ops.expert_gemm_mfma(h, self.w_down, out, perm, offsets, tiles, self.top, planes=True, tile_m=tile_m,
                                 out_scale=w_out)
            return out
        perm, offsets, tiles = ops.route_group(ids.view(-1), self.experts)
        if self.gated:
            gu = torch.empty((slots, 2 * self.inter), dtype=x.dtype, device=x.device)
            ops.expert_gemm(x, self.w_gate_up, gu, perm, offsets, tiles, self.top, gather=True, scale=w_in)
            h = ops.swiglu(gu)
        else:
            h = torch.empty((slots, self.inter), dtype=x.dtype, device=x.device)
            ops.expert_gemm(x, self.w_gate_up, h, perm, offsets, tiles, self.top, gather=True, relu2=True)
        out = torch.empty((self.top, t, self.width), dtype=torch.float32, device=x.device)
        ops.expert_gemm(h, self.w_down, out, perm, offsets, tiles, self.top, gather=False, planes=True, out_scale=w_out)
        return out

    def forward(self, x, ctx):
        ids, weights = ops.route_topk(linear(x, self.w_router, torch.float32), self.top, self.score, self.correction,
                                      self.scale)
        out = self._routed(x, ids, weights)
        if not self.shared:
            return out
        # every token's expert: relu^2 and the token's gate in one pass, then a product like any other that feeds the
        # stream; the norm behind the layer adds it to the routed experts' planes
        u = linear(x, self.w_shared_up, torch.float32)
        h = ops.relu2_gate(u, self.shared, self.shared, x.dtype)
        return WeightedSum([(out, 1.0), (linear_delta(h, self.w_shared_down, None, self.w_shared_down_tiled), 1.0)])


register_feed_forward("routed_experts", RoutedExperts)
