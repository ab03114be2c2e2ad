"""Causal self-attention over the paged cache, with grouped KV heads and an optional window.

Projections without bias (models/src/llama.rs:269-271, 311, 322-325), head split by columns (:273-296), rotation
of q and k (:298-299), keys and values written to the cache before attention (models/src/flash_attention.rs:
360-361), softmax scale 1/sqrt(head size) (models/src/llama.rs:342), query head h on KV head h // (nh/nkv)
(csrc/kernels/flash_fwd_kernel.h:593).  Where the reference runs separate kernels for prompt rows and decode rows
(models/src/flash_attention.rs:380-466), one rule serves here: a token at position p sees keys 0..p (or the
last ``window`` of them) of its own request through the block table.

The three projection matrices are fused into one [(nh + 2 nkv) hd, width] matrix at load time; results equal
the separate products.  When the position encoding rotates whole heads in half-split pairs (i, i + hd/2), the rows
of every q and k head are reordered at load time so that a pair's members leave the projection as neighbours
(2i, 2i + 1): then the projection's own epilogue can rotate q and k and write k and v into the cache, and decode
steps need no kernel between the projection and attention.  Rotated q and cached k are always in their own column
order, whoever rotated them, so any call may read any call's cache.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..kernels import ops
from .base import CacheSpec, Mixer, PositionEncoding, WeightSpec, register_mixer
from .linear import as_tensor, linear, linear_delta


class PagedAttention(Mixer):
    def __init__(self, width: int, num_heads: int, num_kv_heads: int, head_size: int,
                 position: Optional[PositionEncoding] = None, window: Optional[int] = None,
                 scale: Optional[float] = None, chunk: Optional[int] = None, value_size: Optional[int] = None,
                 names=("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight")):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads cannot be grouped over {num_kv_heads} KV heads")
        # ``value_size``: columns of a value head where they differ from a key head's; ``names``: the tensors of the
        # four projections below the part's prefix.  The kernels and the cache see one head size: where keys and values
        # differ, or the size is no multiple of 8, both run as the next multiple of 16 of the larger (``self.hd``;
        # zero rows in the projections, zero columns in the output projection, which changes no score and no output)
        self.hd_in, self.vd_in, self.names = int(head_size), int(value_size or head_size), tuple(names)
        if self.vd_in != self.hd_in or self.hd_in % 8:
            head_size = -(-max(self.hd_in, self.vd_in) // 16) * 16
        # every multiple of 8 up to 256, as the reference's kernels take (csrc/src/lib.rs:136-143, 790)
        if head_size % 8 or not 8 <= head_size <= 256:
            raise ValueError(f"head size {head_size} is not supported: the attention kernels take multiples of 8 "
                             f"from 8 to 256")
        if window is not None and window <= 0:
            raise ValueError("window must be positive")
        if chunk is not None and (chunk <= 0 or window is not None):
            raise ValueError("chunk must be positive, and a layer has a window or chunks, not both")
        self.width, self.nh, self.nkv, self.hd = int(width), int(num_heads), int(num_kv_heads), int(head_size)
        self.position = position
        self.window = window
        # chunk c: the token at p sees keys (p // c) * c .. p only, chunks counted from the request's first position
        self.chunk = chunk
        self.sinks: Optional[torch.Tensor] = None       # float32 [heads]: exp(sinks[h]) joins the softmax denominator
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.hd_in)
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.w_qkv_tiled = self.w_o_tiled = None
        self.act_dtype = torch.float32
        self.paired = False      # q and k columns in pair order (set at load time)
        self.slopes: Optional[torch.Tensor] = None      # per-head bias of the scores by distance, if the encoding has one

    # -- declaration ----------------------------------------------------------------------------------
    def graph_safe(self) -> bool:
        # the kernels take the step from device tensors and from the plan made before the step is recorded
        return self.position is None or self.position.graph_safe()

    def weight_specs(self) -> Dict[str, WeightSpec]:
        n = self.names
        return {n[0]: WeightSpec((self.nh * self.hd_in, self.width)), n[1]: WeightSpec((self.nkv * self.hd_in, self.width)),
                n[2]: WeightSpec((self.nkv * self.vd_in, self.width)), n[3]: WeightSpec((self.width, self.nh * self.vd_in))}

    @staticmethod
    def _pad_heads(w: torch.Tensor, heads: int, size: int, to: int, rows: bool) -> torch.Tensor:
        """``w`` with every head's ``size`` rows (or columns) followed by zeros up to ``to``."""
        if size == to:
            return w
        if rows:
            return torch.nn.functional.pad(w.view(heads, size, w.shape[1]), (0, 0, 0, to - size)).reshape(heads * to, -1)
        return torch.nn.functional.pad(w.view(w.shape[0], heads, size), (0, to - size)).reshape(w.shape[0], heads * to)

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(self.nkv, self.hd, self.window, chunk=self.chunk)

    def load(self, get, device, act_dtype) -> None:
        ws = [self._pad_heads(get(self.names[0]), self.nh, self.hd_in, self.hd, True),
              self._pad_heads(get(self.names[1]), self.nkv, self.hd_in, self.hd, True),
              self._pad_heads(get(self.names[2]), self.nkv, self.vd_in, self.hd, True)]
        dt = ws[0].dtype if all(w.dtype is ws[0].dtype for w in ws) else torch.float32
        if self.position is not None:
            self.position.load(get, device, act_dtype)
        tables = self.position.rotary_tables() if self.position is not None else None
        self.slopes = self.position.score_slopes(self.nh) if self.position is not None else None
        if self.slopes is not None:
            self.slopes = self.slopes.to(device=device, dtype=torch.float32).contiguous()
            if self.slopes.numel() != self.nh:
                raise ValueError(f"score_slopes gave {self.slopes.numel()} slopes for {self.nh} heads")
        self.paired = tables is not None and tables[2] == self.hd
        if self.paired:
            half = self.hd // 2
            order = torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).reshape(-1)   # 0, half, 1, ...
            ws[0] = ws[0].reshape(self.nh, self.hd, self.width)[:, order].reshape(self.nh * self.hd, self.width)
            ws[1] = ws[1].reshape(self.nkv, self.hd, self.width)[:, order].reshape(self.nkv * self.hd, self.width)
        self.w_qkv = torch.cat([w.to(device=device, dtype=dt) for w in ws], dim=0).contiguous()
        self.w_o = self._pad_heads(get(self.names[3]), self.nh, self.vd_in, self.hd, False).to(device).contiguous()
        self.act_dtype = act_dtype
        # second copies in the order in which the kernels of steps of few rows read them
        self.w_qkv_tiled = self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_qkv.dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            if self.paired:
                self.w_qkv_tiled = gemm_bf16.tile_copies_rope(self.w_qkv)
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_qkv, self.w_o))

    def step_planner(self, page_size: int, cache_dtype: torch.dtype):
        """(key, fn(starts, counts, bucket_tokens) -> (int32 array, meta)): the task list of the MFMA attention
        kernels, built once per step on the host and shipped with the step's metadata.  ``bucket_tokens`` is None, or
        for a step that only decodes the context length its plan must serve (a multiple of the runner's bucket)."""
        from ..kernels import attention_bf16
        if self.slopes is not None:
            return None          # scores with a bias take the general kernel, which needs no plan
        if cache_dtype is torch.bfloat16 and self.hd % 16:
            import warnings
            warnings.warn(f"bfloat16 attention with heads of {self.hd} columns runs the general kernel (one wave per "
                          f"token and head), many times slower than the matrix-core kernel, which takes head sizes "
                          f"that are multiples of 16", stacklevel=2)
            return None
        if cache_dtype is torch.bfloat16 and not attention_bf16.page_ok(page_size):
            import warnings
            warnings.warn(f"bfloat16 attention with pages of {page_size} tokens runs the general kernel (one wave per "
                          f"token and head), many times slower than the matrix-core kernel, which needs pages of a "
                          f"multiple of 16 tokens ([cache] block_size = 16, 32, 64, ...)", stacklevel=2)
        if cache_dtype is not torch.bfloat16 or not attention_bf16.page_ok(page_size):
            return None
        group, window, nkv = self.nh // self.nkv, self.span, self.nkv
        cus = torch.cuda.get_device_properties(self.w_o.device).multi_processor_count
        return (attention_bf16.plan_key(group, window, nkv, self.hd),
                lambda starts, counts, bucket: attention_bf16.build_tasks(
                    starts, counts, group, window, bucket, kv_heads=nkv,
                    max_waves=attention_bf16.max_waves_for(self.hd),
                    row_tiles=attention_bf16.max_row_tiles_for(self.hd), head_size=self.hd, compute_units=cus))

    @property
    def span(self) -> int:
        """The mask as the matrix-core kernels and their planner take it: w > 0 a window of the last w keys, -c < 0
        chunks of c positions, 0 all keys."""
        return -self.chunk if self.chunk else (self.window or 0)

    # -- execution ------------------------------------------------------------------------------------
    accepts_begun = True
    takes_sink = True

    def forward(self, x, ctx, cache, sink=None):
        nh, nkv, hd = self.nh, self.nkv, self.hd
        t = x.shape[0]
        writes = cache.writable
        # a call that reads another call's cache needs its queries only
        w = self.w_qkv if writes else self.w_qkv[: nh * hd]
        k_cache, v_cache = cache.k, cache.v
        tables = self.position.rotary_tables() if self.position is not None else None
        qkv = None
        if self.paired and writes and x.dtype is torch.bfloat16 and w.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            qkv = gemm_bf16.try_linear_rope(x, w, ctx.positions, tables[0], tables[1], k_cache, v_cache,
                                            cache.slot_mapping, cache.page_size, nh, nkv, hd,
                                            tiled=self.w_qkv_tiled)
        if qkv is None:
            x = as_tensor(x)
        if qkv is not None:
            pass        # rotated and stored by the product's epilogue
        elif tables is not None or self.position is None:
            raw = linear(x, w)
            cos, sin, rd = tables if tables is not None else (None, None, 0)
            # pair order in, own order out: q cannot be rotated in place then
            qkv = torch.empty((t, nh * hd), dtype=raw.dtype, device=raw.device) if self.paired else raw
            q_out = qkv if self.paired else None
            if writes:
                ops.rope_cache_write(raw, ctx.positions, cos, sin, rd, k_cache, v_cache, cache.slot_mapping,
                                     cache.page_size, nh, nkv, hd, q_out)
            else:
                ops.rope_cache_write(raw, ctx.positions, cos, sin, rd, None, None, None, 1, nh, 0, hd, q_out)
        else:
            qkv = linear(x, w)
            q = qkv[:, : nh * hd].view(t, nh, hd)
            if writes:
                k = qkv[:, nh * hd: (nh + nkv) * hd].view(t, nkv, hd)
                self.position.apply(q, k, ctx.positions)
                ops.rope_cache_write(qkv, ctx.positions, None, None, 0, k_cache, v_cache, cache.slot_mapping,
                                     cache.page_size, nh, nkv, hd)
            else:
                self.position.apply(q, q[:, :0], ctx.positions)
        out = torch.empty((t, nh * hd), dtype=qkv.dtype, device=qkv.device)
        self.attend(qkv, k_cache, v_cache, out, ctx, cache)
        return linear_delta(out, self.w_o, sink, self.w_o_tiled)

    def attend(self, q, k_cache, v_cache, out, ctx, cache) -> None:
        if self.slopes is None and q.dtype is torch.bfloat16 and k_cache.dtype is torch.bfloat16:
            from ..kernels import attention_bf16
            if attention_bf16.try_attention(q, k_cache, v_cache, out, ctx, cache, self.scale, self.span,
                                            self.nh, self.nkv, self.hd, self.sinks):
                return
        ops.paged_attention_generic(q, k_cache, v_cache, out, cache.block_tables, ctx.token_seq, ctx.positions,
                                    self.scale, self.window or 0, cache.page_size, self.nh, self.nkv, self.hd,
                                    self.slopes, self.chunk or 0, self.sinks)


class TiedValueAttention(PagedAttention):
    """Attention whose values are its keys: ``v = W_k x`` as projected, while the keys go on through a norm and the
    rotation.  There is no value projection.

    * q and k are normed over their whole projections (all heads at once) with plain weights ``q.norm``
      [heads * head_size] and ``k.norm`` [kv_heads * head_size], before the rotation;
    * the first ``rotary_dim`` columns of every head are rotated in neighbouring pairs (2i, 2i + 1) by
      position * base^(-2i / rotary_dim), angles in float32, for any position (no table);
    * optional chunks and one learned sink per head (tensor ``sink``), see ``PagedAttention``;
    * any even head size up to 256: one that is no multiple of 16 runs as the next multiple of 16, with zeros in the
      added columns of the queries, of both tiles of the cache and of the output projection (``self.hd`` is the
      size the cache and the attention kernels see, ``self.hd_in`` the checkpoint's).

    Tensors: ``q``, ``k``, ``o`` ([out, in]), ``q.norm``, ``k.norm``, ``sink``.
    """

    def __init__(self, width: int, num_heads: int, num_kv_heads: int, head_size: int, scale: float, norm_eps: float,
                 rotary_base: float, rotary_dim: int, chunk: Optional[int] = None, window: Optional[int] = None,
                 sink: bool = True):
        padded = -(-int(head_size) // 16) * 16      # (multiples of 16: what the matrix-core kernel takes)
        super().__init__(width, num_heads, num_kv_heads, padded, None, window, scale, chunk)
        self.hd_in = self.vd_in = int(head_size)
        if head_size % 2 or rotary_dim % 2 or not 0 <= rotary_dim <= head_size or rotary_dim > 256:
            raise ValueError(f"rotary_dim {rotary_dim} must be even, at most the head size {head_size} and at most 256")
        self.norm_eps, self.rotary_base, self.rotary_dim, self.has_sink = float(norm_eps), float(rotary_base), \
            int(rotary_dim), bool(sink)
        self.w_qk = self.q_norm = self.k_norm = self.inv_freq = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        q, kv = self.nh * self.hd_in, self.nkv * self.hd_in
        specs = {"q": WeightSpec((q, self.width)), "k": WeightSpec((kv, self.width)),
                 "q.norm": WeightSpec((q,), "norm"), "k.norm": WeightSpec((kv,), "norm"),
                 "o": WeightSpec((self.width, q))}
        if self.has_sink:
            specs["sink"] = WeightSpec((self.nh,), "linear", std=1.0)
        return specs

    def load(self, get, device, act_dtype) -> None:
        ws = [get("q"), get("k")]
        dt = ws[0].dtype if ws[0].dtype is ws[1].dtype else torch.float32
        self.w_qk = torch.cat([w.to(device=device, dtype=dt) for w in ws], dim=0).contiguous()
        w_o = get("o").to(device)
        if self.hd != self.hd_in:      # zero columns under the heads' added columns
            w_o = torch.nn.functional.pad(w_o.view(self.width, self.nh, self.hd_in), (0, self.hd - self.hd_in))
        self.w_o = w_o.reshape(self.width, self.nh * self.hd).contiguous()
        f32 = dict(device=device, dtype=torch.float32)
        self.q_norm, self.k_norm = get("q.norm").to(**f32).contiguous(), get("k.norm").to(**f32).contiguous()
        self.sinks = get("sink").to(**f32).contiguous() if self.has_sink else None
        # base^(-2i / dims) in double precision, rounded once to float32
        i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        self.inv_freq = torch.pow(torch.tensor(self.rotary_base, dtype=torch.float64),
                                  -2.0 * i / max(self.rotary_dim, 1)).to(**f32).contiguous()
        self.act_dtype = act_dtype
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_qk, self.w_o))

    accepts_begun = False
    takes_sink = False

    def forward(self, x, ctx, cache, sink=None):
        nh, nkv, hd = self.nh, self.nkv, self.hd
        t = x.shape[0]
        writes = cache.writable
        if not writes:
            raise NotImplementedError("tied-value attention reads only a cache of its own")
        w = self.w_qk
        # the projection leaves in float32: the norm over it and the rotation are float32 work
        qk = linear(x, w, torch.float32)
        q = torch.empty((t, nh * hd), dtype=x.dtype, device=x.device)
        ops.qk_norm_rope(qk, ctx.positions, self.inv_freq, self.rotary_dim, self.q_norm, self.k_norm, self.norm_eps, q,
                         cache.k, cache.v, cache.slot_mapping, cache.page_size, nh, nkv, self.hd_in, hd)
        out = torch.empty((t, nh * hd), dtype=x.dtype, device=x.device)
        self.attend(q, cache.k, cache.v, out, ctx, cache)
        return linear_delta(out, self.w_o, None, self.w_o_tiled)


class LatentAttention(PagedAttention):
    """Attention whose keys and values of every head are products of one small vector per token, the only thing the
    cache keeps:

    * q = W_q x (``heads`` heads of ``head_size``); c = norm(W_dkv x), ``rank`` numbers, RMS-normed with the plain
      weight ``dkv.norm``; per head k = W_uk c and v = W_uv c (``value_size`` columns);
    * no positions are encoded; a token sees every key up to its own; one learned sink per head joins the softmax
      denominator (tensor ``sink``);
    * a head's output is multiplied by sigmoid(W_g x)_head; then W_o.

    The heads' key and value maps are moved to the query's side, ``(W_uk c) . q = c . (W_uk^T q)`` and
    ``sum_j p_j W_uv c_j = W_uv sum_j p_j c_j``: the framework's attention kernels then run with one shared key/value
    head of ``rank`` columns (rounded up to a multiple of 16) whose values are its keys, and a decoded token reads
    ``rank`` numbers per cached token whatever the number of heads.  (The cache keeps c twice, once in the order the
    kernels read keys and once in that of values.)

    Tensors ([out, in]): ``q``, ``dkv``, ``dkv.norm``, ``uk`` [heads * head_size, rank], ``uv`` [heads * value_size,
    rank], ``sink`` [heads], ``g`` [heads, width], ``o`` [width, heads * value_size].
    """

    def __init__(self, width: int, num_heads: int, head_size: int, value_size: int, rank: int, scale: float,
                 norm_eps: float):
        rank_p = -(-int(rank) // 16) * 16
        super().__init__(width, num_heads, 1, rank_p, None, None, scale, None)
        self.qd, self.vd, self.rank, self.norm_eps = int(head_size), int(value_size), int(rank), float(norm_eps)
        self.hd_in = self.vd_in = self.rank
        self.w_in = self.w_uk = self.w_uv = self.c_norm = None
        self.off_c = self.nh * self.qd
        self.off_g = self.off_c + self.rank

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, w, r = self.nh, self.width, self.rank
        return {"q": WeightSpec((h * self.qd, w)), "dkv": WeightSpec((r, w)), "dkv.norm": WeightSpec((r,), "norm"),
                "uk": WeightSpec((h * self.qd, r), std=r ** -0.5), "uv": WeightSpec((h * self.vd, r), std=r ** -0.5),
                "sink": WeightSpec((h,), "linear", std=1.0), "g": WeightSpec((h, w), std=0.1),
                "o": WeightSpec((w, h * self.vd))}

    def load(self, get, device, act_dtype) -> None:
        ws = [get("q"), get("dkv"), get("g")]
        dt = ws[0].dtype if all(w.dtype is ws[0].dtype for w in ws) else torch.float32
        rows = sum(w.shape[0] for w in ws)
        parts = [w.to(device=device, dtype=dt) for w in ws]
        if (-rows) % 64:      # whole tiles for the matrix-core products
            parts.append(torch.zeros(((-rows) % 64, self.width), dtype=dt, device=device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        # per head [out, in]: the key map transposed (it acts on the query), padded to the cache's columns with
        # zero rows; the value map with zero columns under the padding
        uk = get("uk").to(device).view(self.nh, self.qd, self.rank).transpose(1, 2)
        self.w_uk = torch.nn.functional.pad(uk, (0, 0, 0, self.hd - self.rank)).contiguous()
        uv = get("uv").to(device).view(self.nh, self.vd, self.rank)
        self.w_uv = torch.nn.functional.pad(uv, (0, self.hd - self.rank)).contiguous()
        f32 = dict(device=device, dtype=torch.float32)
        self.c_norm = get("dkv.norm").to(**f32).contiguous()
        self.sinks = get("sink").to(**f32).contiguous()
        self.w_o = get("o").to(device).contiguous()
        self.act_dtype = act_dtype
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_uk, self.w_uv, self.w_o))

    accepts_begun = True
    takes_sink = True

    def forward(self, x, ctx, cache, sink=None):
        if not cache.writable:
            raise NotImplementedError("latent attention reads only a cache of its own")
        t = x.shape[0]
        # q, the down projection and the gates leave their product in float32: the norm and the gates are float32 work
        proj = linear(x, self.w_in, torch.float32)
        q, gate = ops.latent_prepare(proj, (0, self.off_c, self.off_g), self.nh, self.qd, self.rank, self.hd,
                                     self.c_norm, self.norm_eps, cache.k, cache.v, cache.slot_mapping,
                                     cache.page_size, x.dtype)
        ql = ops.head_linear(q, self.w_uk, x.dtype)                      # the queries in the latent's columns
        mixed = torch.empty((t, self.nh * self.hd), dtype=x.dtype, device=proj.device)
        self.attend(ql, cache.k, cache.v, mixed, ctx, cache)
        out = ops.head_linear(mixed, self.w_uv, x.dtype, gate)           # the heads' values, gated
        return linear_delta(out, self.w_o, sink, self.w_o_tiled)


class DifferentialAttention(PagedAttention):
    """Attention whose heads each hold two score maps over one set of values and put out the difference of the two
    attentions:

    * q = W_q x has ``heads`` x 2 maps of ``head_size`` columns, k = W_k x has ``kv_heads`` x 2, laid out head by head
      as [map 1 | map 2]; v = W_v x has ``kv_heads`` heads of ``value_size``; query head h reads key/value head
      h // (heads / kv_heads);
    * the first ``rotary_dim`` columns of every map of q and k are turned in half-split pairs (c, c + rotary_dim / 2)
      by position * rotary_base^(-2c / rotary_dim) / ``rotary_factor``; angles are worked out in float32 from the
      position, so there is no table and no largest position;
    * each map is a causal softmax attention a1, a2 with the scale given; o = a1 - lam a2 with
      lam = exp(lq1 . lk1) - exp(lq2 . lk2) + ``diff`` (one number a layer, from four small tensors); o is divided by
      its root mean square over the head's values (eps inside the root, no weight), multiplied by 1 - ``diff`` and
      by sigmoid(W_g x)_head; then W_o.

    How it runs: a key/value head of the cache keeps [k1 | k2] as ONE key of 2 head_size columns and v once, and the
    two maps of a query head are two query heads of that width, map m holding its columns at m * head_size and
    zeros elsewhere, so q' . k' = q_m . k_m.  The framework's attention kernels (matrix-core and general) then serve
    with 2 heads query heads over kv_heads key heads; ``self.hd`` is max(2 head_size, value_size) as a multiple of 16.
    A call that reads another call's cache (``kv_from``) has no k and v tensors and projects q and g only.

    Tensors ([out, in]): ``q``, ``k``, ``v``, ``g`` [heads, width], ``o`` [width, heads * value_size], ``lq1``,
    ``lk1``, ``lq2``, ``lk2`` [head_size].
    """

    def __init__(self, width: int, num_heads: int, num_kv_heads: int, head_size: int, value_size: int, scale: float,
                 diff: float, norm_eps: float, rotary_base: float = 10000.0, rotary_dim: int = 0,
                 rotary_factor: float = 1.0, owns_cache: bool = True):
        wide = -(-max(2 * int(head_size), int(value_size)) // 16) * 16
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads cannot be grouped over {num_kv_heads} KV heads")
        super().__init__(width, 2 * num_heads, num_kv_heads, wide, None, None, scale, None)
        if rotary_dim % 2 or not 0 <= rotary_dim <= head_size or rotary_dim > 256:
            raise ValueError(f"rotary_dim {rotary_dim} must be even, at most the head size {head_size} and at most 256")
        if value_size > 256:
            raise ValueError("values of more than 256 columns a head are not supported")
        self.heads, self.dim, self.vdim = int(num_heads), int(head_size), int(value_size)
        self.hd_in = self.vd_in = wide
        self.diff, self.norm_eps = float(diff), float(norm_eps)
        self.rotary_base, self.rotary_dim, self.rotary_factor = float(rotary_base), int(rotary_dim), float(rotary_factor)
        if not self.rotary_factor > 0:
            raise ValueError("the rotation's scaling factor must be positive")
        self.owns_cache = bool(owns_cache)
        nq = 2 * self.heads * self.dim
        # columns of the fused projection: q, then (with a cache of its own) k and v, then the heads' gates
        self.off_k = nq
        self.off_v = nq + 2 * self.nkv * self.dim
        self.off_g = self.off_v + self.nkv * self.vdim if self.owns_cache else nq
        self.w_in = self.inv_freq = None
        self.lam = 0.0

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, g, d, v, w = self.heads, self.nkv, self.dim, self.vdim, self.width
        specs = {"q": WeightSpec((h * 2 * d, w))}
        if self.owns_cache:
            specs.update({"k": WeightSpec((g * 2 * d, w)), "v": WeightSpec((g * v, w))})
        specs.update({"lq1": WeightSpec((d,), std=0.1), "lk1": WeightSpec((d,), std=0.1),
                      "lq2": WeightSpec((d,), std=0.1), "lk2": WeightSpec((d,), std=0.1),
                      "g": WeightSpec((h, w), std=0.1), "o": WeightSpec((w, h * v))})
        return specs

    def load(self, get, device, act_dtype) -> None:
        ws = [get("q")] + ([get("k"), get("v")] if self.owns_cache else []) + [get("g")]
        dt = ws[0].dtype if all(w.dtype is ws[0].dtype for w in ws) else torch.float32
        rows = sum(w.shape[0] for w in ws)
        parts = [w.to(device=device, dtype=dt) for w in ws]
        if (-rows) % 64:      # whole tiles for the matrix-core products
            parts.append(torch.zeros(((-rows) % 64, self.width), dtype=dt, device=device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_o = get("o").to(device).contiguous()
        # one number a layer, worked out once in float32 as the design asks of everything around the scores
        f32 = lambda n: get(n).to(torch.float32)
        self.lam = float(torch.exp((f32("lq1") * f32("lk1")).sum()) - torch.exp((f32("lq2") * f32("lk2")).sum())
                         + torch.tensor(self.diff, dtype=torch.float32))
        # base^(-2c / dims) / factor in double precision, rounded once to float32
        c = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
        freq = torch.pow(torch.tensor(self.rotary_base, dtype=torch.float64), -2.0 * c / max(self.rotary_dim, 1))
        self.inv_freq = (freq / self.rotary_factor).to(device=device, dtype=torch.float32).contiguous()
        self.act_dtype = act_dtype
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_o))

    accepts_begun = False
    takes_sink = False

    def forward(self, x, ctx, cache, sink=None):
        if cache.writable != self.owns_cache:
            raise RuntimeError("differential attention: a layer with k and v tensors writes its own cache, one "
                               "without reads another layer's")
        t = x.shape[0]
        # the projection leaves in float32: rotation and gates are float32 work
        proj = linear(x, self.w_in, torch.float32)
        q = torch.empty((t, self.nh * self.hd), dtype=x.dtype, device=x.device)
        k, v, slots = (cache.k, cache.v, cache.slot_mapping) if self.owns_cache else (None, None, None)
        gate = ops.diff_prepare(proj, ctx.positions, self.inv_freq, self.rotary_dim, q, k, v, slots, cache.page_size,
                                self.heads, self.nkv, self.dim, self.vdim, self.hd, (self.off_k, self.off_v, self.off_g))
        att = torch.empty((t, self.nh * self.hd), dtype=x.dtype, device=x.device)
        self.attend(q, cache.k, cache.v, att, ctx, cache)
        y = ops.diff_combine(att, gate, self.heads, self.vdim, self.hd, self.lam, self.norm_eps, 1.0 - self.diff, x.dtype)
        return linear_delta(y, self.w_o, None, self.w_o_tiled)


def rotation_frequencies(base: float, dims: int, scaling: Optional[dict] = None):
    """(float32 tensor [dims / 2] of base^(-2i / dims), worked out in double precision and rounded once; the factor on
    cosines and sines).  ``scaling`` = {factor, original, fast, slow} slows the long waves down: with
    where(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(where(fast)), 0), hi = min(ceil(where(slow)),
    dims - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns at
    f_i / factor * ramp_i + f_i (1 - ramp_i), and cosines and sines are multiplied by 0.1 ln(factor) + 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / max(dims, 1))
    mag = 1.0
    if scaling is not None:
        factor, original = float(scaling["factor"]), float(scaling["original"])

        def where(turns: float) -> float:
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(where(float(scaling["fast"]))), 0)
        hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32), mag


class GatedTiedValueAttention(PagedAttention):
    """Attention whose values are its keys as projected (with their bias, before the rotation; no value projection),
    with an output gate per column:

    * q = W_q x + b_q, k = W_k x + b_k; grouped heads (query head h reads key head h // (heads / kv_heads));
    * the first ``rotary_dim`` columns of every q and k head are rotated in half-split pairs (i, i + rotary_dim / 2),
      or neighbouring ones with ``interleaved``, by position * frequency_i, the frequencies optionally slowed down band
      by band (``rotary_scaling``, see ``rotation_frequencies``); angles are float32, worked out from the position;
    * optional chunks or a window; with ``unit_sink`` the softmax denominator holds one more term exp(0) = 1;
    * the heads' outputs are multiplied column by column with sigmoid(W_g x), then W_o x + b_o.

    The output bias is not added here: ``out_bias`` (float32 [width] or None) is for whoever sums the output into the
    stream or norms it.  Head sizes that are no multiple of 16 run as the next multiple (zero columns).

    Tensors ([out, in]): ``q``, ``k``, ``g`` [heads * head_size, width], ``o``; with ``bias`` also ``q.b``, ``k.b``,
    ``o.b``.
    """

    def __init__(self, width: int, num_heads: int, num_kv_heads: int, head_size: int, scale: float,
                 rotary_base: float = 10000.0, rotary_dim: int = 0, rotary_scaling: Optional[dict] = None,
                 interleaved: bool = False, chunk: Optional[int] = None, window: Optional[int] = None,
                 unit_sink: bool = True, bias: bool = True):
        padded = -(-int(head_size) // 16) * 16
        super().__init__(width, num_heads, num_kv_heads, padded, None, window, scale, chunk)
        self.hd_in = self.vd_in = int(head_size)
        if rotary_dim % 2 or not 0 <= rotary_dim <= head_size or rotary_dim > 256:
            raise ValueError(f"rotary_dim {rotary_dim} must be even, at most the head size {head_size} and at most 256")
        self.rotary_base, self.rotary_dim, self.rotary_scaling = float(rotary_base), int(rotary_dim), rotary_scaling
        self.interleaved, self.unit_sink, self.bias = bool(interleaved), bool(unit_sink), bool(bias)
        nq, nk = self.nh * self.hd_in, self.nkv * self.hd_in
        self.off_k, self.off_g = nq, nq + nk
        self.w_in = self.b_q = self.b_k = self.out_bias = self.freq = None
        self.mag = 1.0

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        q, kv, w = self.nh * self.hd_in, self.nkv * self.hd_in, self.width
        specs = {"q": WeightSpec((q, w)), "k": WeightSpec((kv, w)), "g": WeightSpec((q, w)), "o": WeightSpec((w, q))}
        if self.bias:
            specs.update({"q.b": WeightSpec((q,), std=0.1), "k.b": WeightSpec((kv,), std=0.1),
                          "o.b": WeightSpec((w,), std=0.1)})
        return specs

    def load(self, get, device, act_dtype) -> None:
        ws = [get("q"), get("k"), get("g")]
        dt = ws[0].dtype if all(w.dtype is ws[0].dtype for w in ws) else torch.float32
        rows = sum(w.shape[0] for w in ws)
        parts = [w.to(device=device, dtype=dt) for w in ws]
        if (-rows) % 64:      # whole tiles for the matrix-core products
            parts.append(torch.zeros(((-rows) % 64, self.width), dtype=dt, device=device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_o = get("o").to(device).contiguous()
        f32 = dict(device=device, dtype=torch.float32)
        if self.bias:
            self.b_q, self.b_k = get("q.b").to(**f32).contiguous(), get("k.b").to(**f32).contiguous()
            self.out_bias = get("o.b").to(**f32).contiguous()
        freq, self.mag = rotation_frequencies(self.rotary_base, self.rotary_dim, self.rotary_scaling)
        self.freq = freq.to(device).contiguous()
        self.sinks = torch.zeros(self.nh, **f32) if self.unit_sink else None
        self.act_dtype = act_dtype
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_o))

    accepts_begun = False
    takes_sink = False

    def forward(self, x, ctx, cache, sink=None):
        if not cache.writable:
            raise NotImplementedError("tied-value attention reads only a cache of its own")
        t = x.shape[0]
        # the projection leaves in float32: biases, rotation and gates are float32 work
        proj = linear(x, self.w_in, torch.float32)
        q, gate = ops.tied_rope_prepare(proj, (0, self.off_k, self.off_g), self.b_q, self.b_k, ctx.positions, self.freq,
                                        self.rotary_dim, self.interleaved, self.mag, cache.k, cache.v,
                                        cache.slot_mapping, cache.page_size, self.nh, self.nkv, self.hd_in, self.hd,
                                        x.dtype)
        att = torch.empty((t, self.nh * self.hd), dtype=x.dtype, device=x.device)
        self.attend(q, cache.k, cache.v, att, ctx, cache)
        y = ops.gate_mul(att, gate, self.nh, self.hd_in, self.hd)
        return linear_delta(y, self.w_o, None, self.w_o_tiled)


class RotaryLatentAttention(PagedAttention):
    """Attention over one cached latent vector per token, with queries through a latent of their own and a rotated key
    part that all heads share:

    * cq = norm(W_dq x) (``q_rank`` numbers, plain weight ``dq.norm``), q = W_uq cq: per head ``head_size`` columns
      that meet the latent's keys and ``rotary_size`` columns that are rotated;
    * W_dkv x has ``rank`` + ``rotary_size`` rows: the first ``rank``, normed with the plain weight ``dkv.norm``, are
      the latent c; the rest, rotated, is a key part of its own.  Per head k = [W_uk c | that part], v = W_uv c
      (``value_size`` columns); the cache keeps c and the rotated part, nothing else;
    * rotation of neighbouring pairs (2i, 2i + 1) of the first ``rotary_dim`` of the ``rotary_size`` columns by
      position * base^(-2i / rotary_dim), angles in float32 from the position;
    * every earlier key is seen, ordinary softmax, the scale given; the heads' outputs are multiplied column by column
      with sigmoid(W_g x), then W_o.

    As in ``LatentAttention`` the heads' key and value maps act on the query's side: the attention kernels run with
    one shared key head [c | rotated part] of ``rank + rotary_size`` columns (rounded up to a multiple of 16) against
    queries [W_uk^T q_h | rotated q_h], and values [c | 0] of the same width.

    Tensors ([out, in]): ``dq`` [q_rank, width], ``dq.norm``, ``uq`` [heads (head_size + rotary_size), q_rank], ``dkv``
    [rank + rotary_size, width], ``dkv.norm`` [rank], ``uk`` [heads head_size, rank], ``uv`` [heads value_size, rank],
    ``g`` [heads value_size, width], ``o`` [width, heads value_size].
    """

    def __init__(self, width: int, num_heads: int, head_size: int, rotary_size: int, value_size: int, rank: int,
                 q_rank: int, scale: float, norm_eps: float, rotary_base: float = 10000.0,
                 rotary_dim: Optional[int] = None):
        wide = -(-(int(rank) + int(rotary_size)) // 16) * 16
        super().__init__(width, num_heads, 1, wide, None, None, scale, None)
        self.qd, self.rd, self.vd, self.rank, self.q_rank = int(head_size), int(rotary_size), int(value_size),             int(rank), int(q_rank)
        self.rot = self.rd if rotary_dim is None else int(rotary_dim)
        if self.rot % 2 or not 0 <= self.rot <= self.rd or self.rot > 256:
            raise ValueError(f"rotary_dim {self.rot} must be even, at most rotary_size {self.rd} and at most 256")
        self.hd_in = self.vd_in = wide
        self.norm_eps, self.rotary_base = float(norm_eps), float(rotary_base)
        self.off_c = self.q_rank
        self.off_g = self.off_c + self.rank + self.rd
        self.w_in = self.w_uq = self.w_uk = self.w_uv = self.q_norm = self.c_norm = self.freq = None

    def graph_safe(self) -> bool:
        return True

    def weight_specs(self) -> Dict[str, WeightSpec]:
        h, w, r, qr = self.nh, self.width, self.rank, self.q_rank
        return {"dq": WeightSpec((qr, w)), "dq.norm": WeightSpec((qr,), "norm"),
                "uq": WeightSpec((h * (self.qd + self.rd), qr), std=qr ** -0.5),
                "dkv": WeightSpec((r + self.rd, w)), "dkv.norm": WeightSpec((r,), "norm"),
                "uk": WeightSpec((h * self.qd, r), std=r ** -0.5), "uv": WeightSpec((h * self.vd, r), std=r ** -0.5),
                "g": WeightSpec((h * self.vd, w)), "o": WeightSpec((w, h * self.vd))}

    def load(self, get, device, act_dtype) -> None:
        ws = [get("dq"), get("dkv"), get("g")]
        dt = ws[0].dtype if all(w.dtype is ws[0].dtype for w in ws) else torch.float32
        rows = sum(w.shape[0] for w in ws)
        parts = [w.to(device=device, dtype=dt) for w in ws]
        if (-rows) % 64:      # whole tiles for the matrix-core products
            parts.append(torch.zeros(((-rows) % 64, self.width), dtype=dt, device=device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.w_uq = get("uq").to(device).contiguous()
        # per head [out, in]: on the query's side the key map transposed beside an identity that hands the rotated
        # columns through, zero rows up to the cache's width; the value map with zero columns behind the latent's
        uk = get("uk").to(device).view(self.nh, self.qd, self.rank).transpose(1, 2)            # [h, rank, qd]
        wq = torch.zeros((self.nh, self.hd, self.qd + self.rd), dtype=uk.dtype, device=device)
        wq[:, : self.rank, : self.qd] = uk
        wq[:, self.rank: self.rank + self.rd, self.qd:] = torch.eye(self.rd, dtype=uk.dtype, device=device)
        self.w_uk = wq.contiguous()
        uv = get("uv").to(device).view(self.nh, self.vd, self.rank)
        self.w_uv = torch.nn.functional.pad(uv, (0, self.hd - self.rank)).contiguous()
        f32 = dict(device=device, dtype=torch.float32)
        self.q_norm, self.c_norm = get("dq.norm").to(**f32).contiguous(), get("dkv.norm").to(**f32).contiguous()
        self.freq = rotation_frequencies(self.rotary_base, self.rot)[0].to(device).contiguous()
        self.w_o = get("o").to(device).contiguous()
        self.act_dtype = act_dtype
        self.w_o_tiled = None
        if act_dtype is torch.bfloat16 and self.w_o.dtype is torch.bfloat16:
            from ..kernels import gemm_bf16
            self.w_o_tiled = gemm_bf16.tile_copies_resid(self.w_o)

    def device_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_uq, self.w_uk, self.w_uv, self.w_o))

    accepts_begun = False
    takes_sink = False

    def forward(self, x, ctx, cache, sink=None):
        if not cache.writable:
            raise NotImplementedError("latent attention reads only a cache of its own")
        t = x.shape[0]
        # both latents and the gates leave their product in float32: norms, rotation and gates are float32 work
        proj = linear(x, self.w_in, torch.float32)
        cq, gate = ops.latent_rope_prepare(proj, (0, self.off_c, self.off_g), self.q_rank, self.rank, self.rd, self.hd,
                                           self.nh * self.vd, self.q_norm, self.c_norm, self.norm_eps, ctx.positions,
                                           self.freq, self.rot, cache.k, cache.v, cache.slot_mapping, cache.page_size,
                                           x.dtype)
        q = ops.latent_q_rope(linear(cq, self.w_uq, torch.float32), ctx.positions, self.freq, self.rot, self.nh,
                              self.qd, self.rd, x.dtype)
        ql = ops.head_linear(q, self.w_uk, x.dtype)                      # the queries in the cached key's columns
        mixed = torch.empty((t, self.nh * self.hd), dtype=x.dtype, device=proj.device)
        self.attend(ql, cache.k, cache.v, mixed, ctx, cache)
        out = ops.head_linear(mixed, self.w_uv, x.dtype, gate)           # the heads' values, gated column by column
        return linear_delta(out, self.w_o, sink, self.w_o_tiled)


register_mixer("latent_attention", LatentAttention)
register_mixer("differential_attention", DifferentialAttention)
register_mixer("attention", PagedAttention)
register_mixer("tied_value_attention", TiedValueAttention)
register_mixer("gated_tied_value_attention", GatedTiedValueAttention)
register_mixer("rotary_latent_attention", RotaryLatentAttention)
