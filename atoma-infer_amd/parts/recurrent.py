"""Recurrent mixers: a state of fixed size per request in place of a cache that grows.

``GatedDeltaRule``: per head a float32 matrix S [dim, vdim] that every token decays, corrects and reads,

    S <- diag(g) S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q,

* q, k (``kv_heads`` heads of ``dim``) and v (``heads`` heads of ``vdim``) are projections of the input that pass a
  causal depthwise convolution over time (``taps`` taps, the last one the current token's, zeros before the
  request's start) and SiLU; q and k are then scaled to unit length per head (x / sqrt(sum x^2 + 1e-6)), q also by
  dim^-1/2; head h reads q/k head h // (heads / kv_heads);
* beta = sigmoid(W_b x), one per head;
* g = exp(-exp(A_log[h]) * softplus(W_a2 W_a1 x + dt_bias)), one per head and key channel;
* the output: o normed per head over vdim (RMS, weight ``norm`` [vdim] shared by the heads), times
  sigmoid(W_g2 W_g1 x), then W_o.

What is carried from token to token, the state of a request, is S and the last ``taps - 1`` inputs of the
convolution, all float32: one row of the state tensor, [taps - 1][conv channels] followed by [heads][vdim][dim].
Decays, gates of the recurrence, unit lengths and the recurrence itself are float32 in both dtypes; the
projections run in the activation dtype with float32 sums and leave unrounded.

Tensors ([out, in]): ``q``, ``k``, ``v``, ``b``, ``a1``, ``a2``, ``g1``, ``g2``, ``o``; ``q.conv``, ``k.conv``,
``v.conv`` [channels, taps]; ``A_log`` [heads]; ``dt_bias`` [heads * dim]; ``norm`` [vdim].
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import FREE, Mixer, StateSpec, WeightSpec, register_mixer
from .linear import linear, linear_delta


class GatedDeltaRule(Mixer):
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, norm_eps: float,
                 decay_rank: Optional[int] = None, gate_rank: Optional[int] = None):
        # the inner sizes of the two low-rank maps (a1/a2 and g1/g2) are the checkpoint's: None takes whatever
        # the tensors have (the random-weights mode then draws ``DEFAULT_RANK``)
        if heads % kv_heads:
            raise ValueError(f"{heads} heads cannot be grouped over {kv_heads} q/k heads")
        if not 0 < dim <= 256:
            raise ValueError(f"key size {dim} is not supported: the recurrence's kernel takes up to 256")
        if taps < 1:
            raise ValueError("the convolution needs at least the current token's tap")
        self.width, self.heads, self.kv_heads, self.dim, self.vdim = int(width), int(heads), int(kv_heads), int(dim), int(vdim)
        self.taps, self.norm_eps = int(taps), float(norm_eps)
        self.decay_rank = int(decay_rank) if decay_rank else None
        self.gate_rank = int(gate_rank) if gate_rank else None
        self.nqk, self.nv, self.nd = self.kv_heads * self.dim, self.heads * self.vdim, self.heads * self.dim
        self.channels = 2 * self.nqk + self.nv
        # columns of the fused first projection: q, k, v, b, then a1 and g1 (placed at load time)
        self.off_q, self.off_k, self.off_v = 0, self.nqk, 2 * self.nqk
        self.off_b = self.off_v + self.nv
        self.off_a1 = self.off_b + self.heads
        self.off_g1 = None
        self.w_in = self.w_ag = self.w_o = self.w_o_tiled = None
        self.taps_w = self.a_log = self.dt_bias = self.norm_w = None

    def graph_safe(self) -> bool:
        return True     # the kernels take entries, slots and lengths from the step's device tensors

    def weight_specs(self) -> Dict[str, WeightSpec]:
        w, t = self.width, self.taps
        ra, rg = self.decay_rank or FREE, self.gate_rank or FREE
        return {"q": WeightSpec((self.nqk, w)), "q.conv": WeightSpec((self.nqk, t), std=0.5),
                "k": WeightSpec((self.nqk, w)), "k.conv": WeightSpec((self.nqk, t), std=0.5),
                "v": WeightSpec((self.nv, w)), "v.conv": WeightSpec((self.nv, t), std=0.5),
                "b": WeightSpec((self.heads, w), std=0.1), "A_log": WeightSpec((self.heads,), std=0.5, mean=-1.0),
                "norm": WeightSpec((self.vdim,), "norm"),
                "a1": WeightSpec((ra, w), std=0.1), "a2": WeightSpec((self.nd, ra), std=0.3),
                "dt_bias": WeightSpec((self.nd,), std=1.0, mean=-2.0),
                "g1": WeightSpec((rg, w), std=0.1), "g2": WeightSpec((self.nv, rg), std=0.3),
                "o": WeightSpec((w, self.nv))}

    def state_spec(self) -> StateSpec:
        return StateSpec(((self.taps - 1) * self.channels + self.heads * self.vdim * self.dim,), "float32")

    def load(self, get, device, act_dtype) -> None:
        ws = [get(n) for n in ("q", "k", "v", "b", "a1", "g1")]
        self.decay_rank, self.gate_rank = ws[4].shape[0], ws[5].shape[0]
        self.off_g1 = self.off_a1 + self.decay_rank
        dt = ws[0].dtype if all(w.dtype is ws[0].dtype for w in ws) else torch.float32
        rows = sum(w.shape[0] for w in ws)
        pad = (-rows) % 64      # whole tiles for the matrix-core products
        parts = [w.to(device=device, dtype=dt) for w in ws]
        if pad:
            parts.append(torch.zeros((pad, self.width), dtype=dt, device=device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        a2, g2 = get("a2"), get("g2")
        if a2.shape[1] != self.decay_rank or g2.shape[1] != self.gate_rank:
            raise ValueError(f"the halves of a low-rank map do not fit: a1 {tuple(ws[4].shape)} and a2 "
                             f"{tuple(a2.shape)}, g1 {tuple(ws[5].shape)} and g2 {tuple(g2.shape)}")
        # the second halves of both low-rank maps as one matrix, [[a2, 0], [0, g2]], for one product over the
        # neighbouring columns of a1's and g1's results (the zeros add nothing)
        dt2 = a2.dtype if a2.dtype is g2.dtype else torch.float32
        self.w_ag = torch.zeros((self.nd + self.nv, self.decay_rank + self.gate_rank), dtype=dt2, device=device)
        self.w_ag[: self.nd, : self.decay_rank] = a2.to(device=device, dtype=dt2)
        self.w_ag[self.nd:, self.decay_rank:] = g2.to(device=device, dtype=dt2)
        self.w_o = get("o").to(device).contiguous()
        f32 = dict(device=device, dtype=torch.float32)
        self.taps_w = torch.cat([get(n + ".conv").to(**f32) for n in ("q", "k", "v")], dim=0).contiguous()
        self.a_log, self.dt_bias = get("A_log").to(**f32).contiguous(), get("dt_bias").to(**f32).contiguous()
        self.norm_w = get("norm").to(**f32).contiguous()
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_ag, self.w_o))

    def forward(self, x, ctx, cache):
        state = cache.state
        proj = linear(x, self.w_in, torch.float32)
        # the second halves of the two low-rank maps read their columns of the float32 projection as they are
        low = proj[:, self.off_a1: self.off_g1 + self.gate_rank]
        pre = ops.lowrank_up(low, self.w_ag) if x.shape[0] <= ops.LOWRANK_UP_MAX_TOKENS else \
            linear(low, self.w_ag, torch.float32)
        dt_pre, gate_pre = pre[:, : self.nd], pre[:, self.nd:]
        qn, kn, vn, beta, decay, kq = ops.delta_prepare(
            proj, (self.off_q, self.off_k, self.off_v, self.off_b), self.heads, self.kv_heads, self.dim, self.vdim,
            self.taps, ctx.token_seq, ctx.q_start, ctx.state_slots, state, self.taps_w, dt_pre, self.dt_bias, self.a_log)
        o = ops.delta_scan(qn, kn, vn, beta, decay, kq, self.heads, self.kv_heads, self.dim, self.vdim, self.taps,
                           ctx.q_start, ctx.state_slots, state)
        y = ops.delta_out(o, gate_pre, self.norm_w, self.norm_eps, self.heads, self.vdim, x.dtype)
        return linear_delta(y, self.w_o, None, self.w_o_tiled)


class StateSpaceDuality(Mixer):
    """A selective state-space recurrence with one scalar decay per head (the Mamba-2 form): per head a float32 matrix
    S [state, vdim],

        S <- exp(-exp(A_log) dt) S + dt B x^T;   y = S^T C + D x;   dt = softplus(W_dt h + dt_bias),

    * one input projection whose rows are laid out [z: inner | x: inner | B: groups * state | C: groups * state |
      dt: heads], inner = heads * vdim; x, B and C together pass a causal depthwise convolution over time (``taps``
      taps with bias, the last one the current token's, zeros before the request's start) and SiLU; head h reads the B
      and C of group h // (heads / groups);
    * the output: y * silu(z), RMS-normed in ``norm_groups`` equal parts of the row, times ``norm``, then W_o.

    What is carried from token to token, the state of a request, is S and the last ``taps - 1`` inputs of the
    convolution, all float32: one row of the state tensor, [taps - 1][conv channels] followed by [heads][vdim][state].
    Step sizes, decays, the convolution and the recurrence are float32 in both dtypes; the projections run in the
    activation dtype with float32 sums and leave unrounded.

    Tensors: ``in`` [2 inner + 2 groups state + heads, width], ``conv`` [channels, taps], ``conv.b`` [channels],
    ``dt_bias``, ``A_log``, ``D`` [heads], ``norm`` [inner], ``o`` [width, inner].
    """

    def __init__(self, width: int, heads: int, groups: int, vdim: int, state: int, taps: int, norm_groups: int,
                 norm_eps: float):
        if heads % groups:
            raise ValueError(f"{heads} heads cannot be grouped over {groups} groups of B and C")
        if not 0 < state <= 256:
            raise ValueError(f"state size {state} is not supported: the recurrence's kernel takes up to 256")
        if not 1 <= taps <= 64:
            raise ValueError("the convolution takes 1 to 64 taps")
        self.width, self.heads, self.groups, self.vdim, self.n = int(width), int(heads), int(groups), int(vdim), int(state)
        self.taps, self.norm_groups, self.norm_eps = int(taps), int(norm_groups), float(norm_eps)
        self.inner = self.heads * self.vdim
        if self.inner % self.norm_groups:
            raise ValueError(f"{norm_groups} norm groups do not divide the inner width {self.inner}")
        self.channels = self.inner + 2 * self.groups * self.n
        self.off_z, self.off_x, self.off_dt = 0, self.inner, self.inner + self.channels
        self.w_in = self.w_o = self.w_o_tiled = None
        self.taps_w = self.conv_b = self.a_log = self.dt_bias = self.d_skip = self.norm_w = None

    def graph_safe(self) -> bool:
        return True     # the kernels take entries, slots and lengths from the step's device tensors

    def weight_specs(self) -> Dict[str, WeightSpec]:
        w, h = self.width, self.heads
        return {"in": WeightSpec((self.off_dt + h, w), std=0.05), "conv": WeightSpec((self.channels, self.taps), std=0.5),
                "conv.b": WeightSpec((self.channels,), std=0.1), "dt_bias": WeightSpec((h,), std=1.0, mean=-1.0),
                "A_log": WeightSpec((h,), std=0.5, mean=-0.5), "D": WeightSpec((h,), std=0.5, mean=1.0),
                "norm": WeightSpec((self.inner,), "norm"), "o": WeightSpec((w, self.inner))}

    def state_spec(self) -> StateSpec:
        return StateSpec(((self.taps - 1) * self.channels + self.heads * self.vdim * self.n,), "float32")

    def load(self, get, device, act_dtype) -> None:
        w_in = get("in").to(device)
        pad = (-w_in.shape[0]) % 64      # whole tiles for the matrix-core products
        if pad:
            w_in = torch.cat([w_in, torch.zeros((pad, self.width), dtype=w_in.dtype, device=device)], dim=0)
        self.w_in = w_in.contiguous()
        self.w_o = get("o").to(device).contiguous()
        f32 = dict(device=device, dtype=torch.float32)
        self.taps_w, self.conv_b = get("conv").to(**f32).contiguous(), get("conv.b").to(**f32).contiguous()
        self.a_log, self.dt_bias = get("A_log").to(**f32).contiguous(), get("dt_bias").to(**f32).contiguous()
        self.d_skip, self.norm_w = get("D").to(**f32).contiguous(), get("norm").to(**f32).contiguous()
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_o))

    accepts_begun = True
    takes_sink = True

    def forward(self, x, ctx, cache, sink=None):
        state = cache.state
        dims = (self.heads, self.groups, self.vdim, self.n, self.taps)
        proj = linear(x, self.w_in, torch.float32)
        xbc, dt, decay = ops.ssd_prepare(proj, (self.off_z, self.off_x, self.off_dt), *dims, ctx.token_seq, ctx.q_start,
                                         ctx.state_slots, state, self.taps_w, self.conv_b, self.dt_bias, self.a_log)
        ops.ssd_conv_state(proj, self.off_x, *dims, ctx.q_start, ctx.state_slots, state)
        y = ops.ssd_scan(xbc, dt, decay, self.a_log, self.d_skip, *dims, ctx.q_start, ctx.state_slots, state,
                         counts=ctx.h_counts)
        u = ops.ssd_out(y, proj, self.off_z, self.norm_w, self.norm_eps, self.norm_groups, x.dtype)
        return linear_delta(u, self.w_o, sink, self.w_o_tiled)


class MinGRU(Mixer):
    """A gated recurrence whose gates read the current token only (the minGRU form): per channel

        z = sigmoid(W_z h + b_z);   u = W_x h + b_x;   c = u + 1/2 where u >= 0, sigmoid(u) where u < 0;
        S <- (1 - z) S + z c;       out = W_o (S * silu(W_g h)),

    ``inner`` channels.  A request's state is S, one float32 row, zero at its start.  Gates, candidate and S are
    float32 in both dtypes; the three input projections are one product in the activation dtype with float32 sums
    that leaves unrounded.  Since the step is linear in S, entries of many tokens are walked in stretches side by
    side (``ops.mingru_plan``, made once per step on the host), and decoded tokens by the plain walk.

    Tensors ([out, in]): ``z``, ``x``, ``g`` [inner, width], ``z.b``, ``x.b`` [inner], ``o`` [width, inner].
    """

    def __init__(self, width: int, inner: int):
        if inner <= 0:
            raise ValueError("the recurrence needs at least one channel")
        self.width, self.inner = int(width), int(inner)
        self.off_x, self.off_g = self.inner, 2 * self.inner
        self.w_in = self.w_o = self.w_o_tiled = self.b_z = self.b_x = None

    def graph_safe(self) -> bool:
        return True     # entries, slots and lengths come from the step's device tensors, stretches from its plan

    def weight_specs(self) -> Dict[str, WeightSpec]:
        w, n = self.width, self.inner
        return {"z": WeightSpec((n, w), std=0.08), "z.b": WeightSpec((n,), std=0.5),
                "x": WeightSpec((n, w), std=0.08), "x.b": WeightSpec((n,), std=0.5),
                "g": WeightSpec((n, w), std=0.08), "o": WeightSpec((w, n))}

    def state_spec(self) -> StateSpec:
        return StateSpec((self.inner,), "float32")

    def load(self, get, device, act_dtype) -> None:
        ws = [get("z"), get("x"), get("g")]
        dt = ws[0].dtype if all(w.dtype is ws[0].dtype for w in ws) else torch.float32
        parts = [w.to(device=device, dtype=dt) for w in ws]
        if (-3 * self.inner) % 64:      # whole tiles for the matrix-core products
            parts.append(torch.zeros(((-3 * self.inner) % 64, self.width), dtype=dt, device=device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_o = get("o").to(device).contiguous()
        f32 = dict(device=device, dtype=torch.float32)
        self.b_z, self.b_x = get("z.b").to(**f32).contiguous(), get("x.b").to(**f32).contiguous()
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_o))

    def step_planner(self, page_size: int, cache_dtype: torch.dtype):
        """(key, fn(starts, counts, bucket_tokens) -> (int32 array, stretches)): the stretches of long entries."""
        import numpy as np
        cus = torch.cuda.get_device_properties(self.w_o.device).multi_processor_count
        blocks = -(-self.inner // 256)

        def plan(starts, counts, bucket):
            got = ops.mingru_plan(counts, self.inner, cus)
            return got if got is not None else (np.zeros(0, dtype=np.int32), 0)
        return ("mingru_stretches", blocks), plan

    def forward(self, x, ctx, cache):
        proj = linear(x, self.w_in, torch.float32)
        blocks = -(-self.inner // 256)
        plan = getattr(ctx, "plans", {}).get(("mingru_stretches", blocks))
        if plan is None and getattr(ctx, "h_counts", None) is not None:
            # a caller without a step planner (a kernel test): plan here and now
            got = ops.mingru_plan(ctx.h_counts, self.inner)
            if got is not None:
                plan = (torch.from_numpy(got[0]).to(x.device), got[1])
        y = ops.mingru(proj, self.off_x, self.off_g, self.inner, self.b_z, self.b_x, ctx.q_start, ctx.state_slots,
                       cache.state, x.dtype, plan)
        return linear_delta(y, self.w_o, None, self.w_o_tiled)


class LightningAttention(Mixer):
    """Linear attention with one fixed decay per head: q = silu(W_q x), k = silu(W_k x) (``heads`` x ``dim``),
    v = silu(W_v x) (``heads`` x ``vdim``); per head

        S <- decay_h S + k v^T;   o = S^T q      (no other scale),

    the heads' outputs normed together (RMS, plain weight ``norm``), multiplied by sigmoid(W_g x) and projected by W_o.
    A request's state is S, float32 [heads][vdim][dim], zero at its start.  The four input projections are one product
    with float32 sums that leaves unrounded; SiLU, the recurrence, the norm and the gate are float32 in both dtypes.
    With bfloat16 activations, entries of ``CHUNKED_FROM`` tokens or more run 64 tokens at a time on the matrix cores,
    q, k and v rounded to bfloat16 there (as activations are), the state and every sum still float32.

    Tensors ([out, in]): ``q``, ``k`` [heads dim, width], ``v``, ``g`` [heads vdim, width], ``norm`` [heads vdim],
    ``o`` [width, heads vdim].
    """

    CHUNKED_FROM = 24

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay, norm_eps: float):
        decay = [float(d) for d in decay]
        if len(decay) != heads:
            raise ValueError(f"{len(decay)} decays for {heads} heads")
        if dim > 256:
            raise ValueError("key sizes beyond 256 are not supported by the recurrence's kernel")
        self.width, self.heads, self.dim, self.vdim, self.decay_list = int(width), int(heads), int(dim), int(vdim), decay
        self.norm_eps = float(norm_eps)
        nq, nv = self.heads * self.dim, self.heads * self.vdim
        self.off_k, self.off_v, self.off_g = nq, 2 * nq, 2 * nq + nv
        self.w_in = self.w_o = self.w_o_tiled = self.norm_w = self.decay = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        w, nq, nv = self.width, self.heads * self.dim, self.heads * self.vdim
        return {"q": WeightSpec((nq, w), std=0.08), "k": WeightSpec((nq, w), std=0.08),
                "v": WeightSpec((nv, w), std=0.08), "g": WeightSpec((nv, w), std=0.08),
                "norm": WeightSpec((nv,), "norm"), "o": WeightSpec((w, nv))}

    def state_spec(self) -> StateSpec:
        return StateSpec((self.heads * self.vdim * self.dim,), "float32")

    def load(self, get, device, act_dtype) -> None:
        ws = [get("q"), get("k"), get("v"), get("g")]
        dt = ws[0].dtype if all(w.dtype is ws[0].dtype for w in ws) else torch.float32
        rows = sum(w.shape[0] for w in ws)
        parts = [w.to(device=device, dtype=dt) for w in ws]
        if (-rows) % 64:      # whole tiles for the matrix-core products
            parts.append(torch.zeros(((-rows) % 64, self.width), dtype=dt, device=device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_o = get("o").to(device).contiguous()
        f32 = dict(device=device, dtype=torch.float32)
        self.norm_w = get("norm").to(**f32).contiguous()
        self.decay = torch.tensor(self.decay_list, dtype=torch.float64).to(**f32).contiguous()
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_o))

    def forward(self, x, ctx, cache):
        proj = linear(x, self.w_in, torch.float32)
        chunked = self.CHUNKED_FROM if (x.dtype is torch.bfloat16 and self.dim % 32 == 0 and self.dim <= 128
                                        and min(self.decay_list) > 0.0) else 0
        # which of the two kernels a step needs follows from its entries' lengths, as its graph's key does
        counts = getattr(ctx, "h_counts", None)
        scan = True
        if chunked and counts is not None and len(counts):
            scan = int(counts.min()) < chunked
            if int(counts.max()) < chunked:
                chunked = 0
        o = ops.lightning_scan(proj, (0, self.off_k, self.off_v), ctx.q_start, ctx.state_slots, cache.state, self.decay,
                               self.heads, self.dim, self.vdim, chunked, scan)
        y = ops.lightning_out(o, proj, self.off_g, self.norm_w, self.norm_eps, x.dtype)
        return linear_delta(y, self.w_o, None, self.w_o_tiled)


class GatedLinearRecurrence(Mixer):
    """Griffin's recurrent block around a real-gated linear recurrent unit, ``inner`` channels:

        g = gelu_tanh(W_y x + b_y);   u = conv(W_x x + b_x)     (causal, per channel, ``taps`` taps, bias, no activation)
        r = sigmoid(Ra u + ba);   i = sigmoid(Ri u + bi)        (Ra, Ri: ``blocks`` square blocks on the diagonal)
        a = exp(-8 r softplus(lam));   S <- a S + sqrt(1 - a^2) i u;   out = W_o (S g).

    A request's state is the convolution's last ``taps - 1`` inputs and S, float32, zero at its start.  The two input
    projections are one product with float32 sums that leaves unrounded; everything behind it, the gates' products
    included, is float32 in both dtypes.  The step is linear in S, so entries of many tokens are walked in stretches
    side by side (the plan of ``ops.mingru_plan``), decoded tokens by the plain walk.

    Tensors ([out, in]): ``y``, ``x`` [inner, width] with ``y.b``, ``x.b``; ``conv`` [inner, taps] (last column: the
    current token), ``conv.b``; ``ra``, ``ri`` [blocks, inner / blocks, inner / blocks] with ``ra.b``, ``ri.b``
    [blocks, inner / blocks]; ``lam`` [inner]; ``o`` [width, inner].
    """

    def __init__(self, width: int, inner: int, blocks: int, taps: int):
        if inner <= 0 or blocks <= 0 or inner % blocks or not 1 <= taps <= 64:
            raise ValueError(f"a recurrence of {inner} channels in {blocks} blocks with {taps} taps is not supported")
        self.width, self.inner, self.blocks, self.taps = int(width), int(inner), int(blocks), int(taps)
        self.bs = self.inner // self.blocks
        self.w_in = self.w_gates = self.w_o = self.w_o_tiled = None
        self.b_y = self.b_x = self.conv = self.conv_b = self.b_a = self.b_i = self.sp = None
        self.out_bias = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        w, n, b, bs, k = self.width, self.inner, self.blocks, self.bs, self.taps
        return {"y": WeightSpec((n, w), std=0.08), "y.b": WeightSpec((n,), std=0.3),
                "x": WeightSpec((n, w), std=0.08), "x.b": WeightSpec((n,), std=0.3),
                "conv": WeightSpec((n, k), std=0.4), "conv.b": WeightSpec((n,), std=0.1),
                "ra": WeightSpec((b, bs, bs), std=bs ** -0.5), "ra.b": WeightSpec((b, bs), std=0.5),
                "ri": WeightSpec((b, bs, bs), std=bs ** -0.5), "ri.b": WeightSpec((b, bs), std=0.5),
                "lam": WeightSpec((n,), std=1.0, mean=-1.0), "o": WeightSpec((w, n))}

    def state_spec(self) -> StateSpec:
        return StateSpec((self.taps * self.inner,), "float32")

    def load(self, get, device, act_dtype) -> None:
        ws = [get("y"), get("x")]
        dt = ws[0].dtype if ws[0].dtype is ws[1].dtype else torch.float32
        parts = [w.to(device=device, dtype=dt) for w in ws]
        if (-2 * self.inner) % 64:      # whole tiles for the matrix-core products
            parts.append(torch.zeros(((-2 * self.inner) % 64, self.width), dtype=dt, device=device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_o = get("o").to(device).contiguous()
        f32 = dict(device=device, dtype=torch.float32)
        vec = lambda name: get(name).to(**f32).reshape(-1).contiguous()
        self.b_y, self.b_x, self.conv_b = vec("y.b"), vec("x.b"), vec("conv.b")
        self.conv = get("conv").to(**f32).contiguous()
        self.b_a, self.b_i = vec("ra.b"), vec("ri.b")
        # per block the rows of Ra, then those of Ri: one product per block gives [r | i] before their biases
        self.w_gates = torch.cat([get("ra").to(**f32), get("ri").to(**f32)], dim=1).contiguous()
        # softplus(lam) in float32, once: log(1 + exp(lam)) in its stable form
        lam = vec("lam")
        self.sp = (torch.clamp(lam, min=0.0) + torch.log1p(torch.exp(-lam.abs()))).contiguous()
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_gates, self.w_o))

    MIN_STRETCH = 32

    def _plan_key(self):
        return ("rglru_stretches", -(-self.inner // 256))

    def step_planner(self, page_size: int, cache_dtype: torch.dtype):
        import numpy as np
        cus = torch.cuda.get_device_properties(self.w_o.device).multi_processor_count

        def plan(starts, counts, bucket):
            got = ops.mingru_plan(counts, self.inner, cus, self.MIN_STRETCH)
            return got if got is not None else (np.zeros(0, dtype=np.int32), 0)
        return self._plan_key(), plan

    def forward(self, x, ctx, cache):
        proj = linear(x, self.w_in, torch.float32)
        u, g = ops.rglru_conv(proj, 0, self.inner, self.b_y, self.b_x, self.conv, self.conv_b, ctx.token_seq,
                              ctx.q_start, ctx.state_slots, cache.state, self.inner, self.taps)
        gates = ops.head_linear(u, self.w_gates, torch.float32)
        plan = getattr(ctx, "plans", {}).get(self._plan_key())
        if plan is None and getattr(ctx, "h_counts", None) is not None:
            # a caller without a step planner: plan here and now
            got = ops.mingru_plan(ctx.h_counts, self.inner, min_length=self.MIN_STRETCH)
            if got is not None:
                plan = (torch.from_numpy(got[0]).to(x.device), got[1])
        y = ops.rglru_scan(gates, u, g, self.b_a, self.b_i, self.sp, ctx.q_start, ctx.state_slots, cache.state,
                           self.blocks, self.taps, x.dtype, plan)
        return linear_delta(y, self.w_o, None, self.w_o_tiled)


register_mixer("gated_delta_rule", GatedDeltaRule)
register_mixer("mingru", MinGRU)
register_mixer("lightning_attention", LightningAttention)
register_mixer("gated_linear_recurrence", GatedLinearRecurrence)
register_mixer("state_space_duality", StateSpaceDuality)
