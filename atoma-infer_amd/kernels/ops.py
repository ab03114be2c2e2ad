"""Python face of the HIP kernels: argument checks on the host, then one C call per op on the current stream.

Every function takes device tensors and writes into tensors the caller passes or that it allocates with torch
(torch is the allocator and the stream owner; it computes nothing here).  Shapes, strides and dtypes are checked
before a launch, because a kernel that reads outside a tensor can take the GPU down.  A missing or unbuildable
library raises ``KernelBuildError``; there is no other code path.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .library import load_hip_module

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"{what}: dtype {t.dtype} is not supported (float32 or bfloat16)") from None


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream of the current device as the kernels' launch argument.  Asked for at every launch (a
    graph capture changes it); the raw accessor costs a fraction of a microsecond, the public one several."""
    if _raw_stream is not None and _raw_device is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc: int, op: str):
    if rc == 0:
        return
    if rc == -2:
        raise KernelError(f"{op}: unsupported combination of element types")
    if rc == -3:
        raise KernelError(f"{op}: the kernel refuses these sizes")
    raise KernelError(f"{op}: HIP error {rc}")


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _dev(*ts):
    for t in ts:
        if t is not None:
            _need(t.is_cuda, "kernels run on device tensors only; got a CPU tensor")


def _i32(t: torch.Tensor, what: str, n: Optional[int] = None):
    _need(t.dtype is torch.int32 and t.is_contiguous(), f"{what} must be a contiguous int32 tensor")
    if n is not None:
        _need(t.numel() >= n, f"{what} has {t.numel()} entries, {n} are needed")


_core = None


def core():
    global _core
    if _core is None:
        _core = load_hip_module("core")
    return _core


# ------------------------------------------------------------------------------------------------------------

def embed(tokens: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = table[tokens[t]] as float32; a token outside the table gives a row of NaN."""
    _dev(tokens, table)
    _i32(tokens, "tokens")
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [vocab, width]")
    n, width = tokens.numel(), table.shape[1]
    if out is None:
        out = torch.empty((n, width), dtype=torch.float32, device=table.device)
    _need(out.dtype is torch.float32 and out.is_contiguous() and tuple(out.shape) == (n, width), "embed: bad out")
    _check(core().atoma_embed(_p(tokens), _p(table), _code(table, "embedding table"), _p(out), n, width,
                              table.shape[0], _stream()), "embed")
    return out


def embed_begin_norm(tokens: torch.Tensor, table: torch.Tensor, gamma: torch.Tensor):
    """The embedding gather with a norm begun, for at most 16 tokens: (resid float32 [T, W], u bfloat16 [T, W] =
    resid * gamma, ss float32 [1, 16] the rows' sums of squares).  A product finishes the norm (gemm_bf16)."""
    _dev(tokens, table, gamma)
    _i32(tokens, "tokens")
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [vocab, width]")
    n, width = tokens.numel(), table.shape[1]
    _need(0 < n <= 16, "embed_begin_norm takes at most 16 tokens")
    _need(gamma.is_contiguous() and gamma.numel() == width, "norm weight must have one entry per column")
    resid = torch.empty((n, width), dtype=torch.float32, device=table.device)
    u = torch.empty((n, width), dtype=torch.bfloat16, device=table.device)
    ss = torch.empty((1, 16), dtype=torch.float32, device=table.device)
    _check(core().atoma_embed_begin_norm(_p(tokens), _p(table), _code(table, "embedding table"), _p(resid), _p(gamma),
                                         _code(gamma, "norm weight"), _p(u), _p(ss), n, width, table.shape[0],
                                         _stream()), "embed_begin_norm")
    return resid, u, ss


def finish_norm(u: torch.Tensor, ss: torch.Tensor, eps: float, width: int) -> torch.Tensor:
    """u [T <= 16, W] bfloat16 divided by sqrt(sum_p ss[p, row] / width + eps), row by row, as bfloat16."""
    _dev(u, ss)
    _need(u.dtype is torch.bfloat16 and u.dim() == 2 and u.is_contiguous() and u.shape[0] <= 16, "finish_norm: bad u")
    _need(ss.dtype is torch.float32 and ss.dim() == 2 and ss.shape[1] == 16 and ss.is_contiguous(),
          "finish_norm: shares must be float32 [parts, 16]")
    out = torch.empty_like(u)
    _check(core().atoma_finish_norm(_p(u), _p(ss), ss.shape[0], ctypes.c_float(eps), _p(out), u.shape[0], u.shape[1],
                                    _stream()), "finish_norm")
    return out


def add_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """resid += delta (in place, float32); return rmsnorm(resid) * weight in ``out_dtype``.

    With ``rows`` (int32 row numbers) only those rows are summed and normed, into a result of len(rows) rows,
    and resid is left as it is.
    """
    _dev(resid, delta, weight, rows)
    _need(resid.dtype is torch.float32 and resid.dim() == 2 and resid.is_contiguous(), "resid must be float32 [T, W]")
    t, width = resid.shape
    _need(weight.is_contiguous() and weight.numel() == width, "norm weight must have one entry per column")
    planes, plane_stride = 1, 0
    if delta is not None:
        if delta.dim() == 3:  # planes of a K-split product, summed here
            planes, plane_stride = delta.shape[0], t * width
            _need(delta.is_contiguous() and tuple(delta.shape[1:]) == (t, width), "delta planes must match resid")
        else:
            _need(delta.is_contiguous() and tuple(delta.shape) == (t, width), "delta must match resid")
    n = t
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    if out is None:
        out = torch.empty((n, width), dtype=out_dtype, device=resid.device)
    _need(out.is_contiguous() and tuple(out.shape) == (n, width) and out.dtype is out_dtype, "add_rmsnorm: bad out")
    _check(core().atoma_add_rmsnorm(_p(resid), _p(delta), _code(delta, "delta") if delta is not None else F32,
                                    _p(weight), _code(weight, "norm weight"), _p(out), _code(out, "out"), _p(rows),
                                    n, width, ctypes.c_float(eps), planes, ctypes.c_size_t(plane_stride),
                                    _stream()), "add_rmsnorm")
    return out


def rope_cache_write(qkv: torch.Tensor, positions: torch.Tensor, cos: Optional[torch.Tensor],
                     sin: Optional[torch.Tensor], rotary_dim: int, kcache: Optional[torch.Tensor],
                     vcache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor], page_size: int, nh: int,
                     nkv: int, hd: int, q_out: Optional[torch.Tensor] = None) -> None:
    """Rotate q and k of ``qkv`` [T, (nh + 2 nkv) hd] (q in place), store rotated k and v at ``slot_mapping``.

    kcache and vcache are [pages, nkv, page_size * hd] tiles (order: cache/layout.py).  Null caches: rotate q only.
    With ``q_out`` [T, nh hd] the members of pair i arrive as columns 2i and 2i + 1 of a q or k head (rows of the
    projection reordered at load time); the rotated q is written to ``q_out`` and k to the cache in their own
    column order, and ``qkv`` is left as it is.
    """
    _dev(qkv, positions, cos, sin, kcache, vcache, slot_mapping)
    t = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] >= (nh + 2 * nkv) * hd, "qkv: bad shape")
    _i32(positions, "positions", t)
    if cos is not None:
        _need(sin is not None and cos.dtype is torch.float32 and sin.dtype is torch.float32 and cos.is_contiguous()
              and sin.is_contiguous() and cos.shape == sin.shape and cos.shape[1] == rotary_dim // 2,
              "rotary tables must be float32 [positions, rotary_dim/2]")
    cache_code = _code(qkv, "qkv")
    if q_out is not None:
        _dev(q_out)
        _need(q_out.dtype is qkv.dtype and q_out.dim() == 2 and q_out.stride(1) == 1 and q_out.shape[0] == t
              and q_out.shape[1] >= nh * hd and cos is not None and rotary_dim == hd,
              "q_out must be [T, nh hd] of qkv's dtype, with the whole head rotated")
    if kcache is not None:
        _need(vcache is not None and slot_mapping is not None, "cache write needs k, v and slots")
        _i32(slot_mapping, "slot_mapping", t)
        pages = kcache.shape[0]
        _need(kcache.is_contiguous() and vcache.is_contiguous() and tuple(kcache.shape) == (pages, nkv, page_size * hd)
              and tuple(vcache.shape) == (pages, nkv, page_size * hd) and kcache.dtype is vcache.dtype,
              "cache tensors must be [pages, nkv, page_size * hd] tiles")
        cache_code = _code(kcache, "cache")
    _check(core().atoma_rope_cache_write(_p(qkv), _code(qkv, "qkv"), qkv.stride(0), _p(positions), _p(cos), _p(sin),
                                         rotary_dim, _p(kcache), _p(vcache), cache_code, _p(slot_mapping), page_size,
                                         t, nh, nkv, hd, _p(q_out), q_out.stride(0) if q_out is not None else 0,
                                         _stream()), "rope_cache_write")


def paged_attention_generic(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, out: torch.Tensor,
                            block_tables: torch.Tensor, token_seq: torch.Tensor, positions: torch.Tensor,
                            scale: float, window: int, page_size: int, nh: int, nkv: int, hd: int,
                            slopes: Optional[torch.Tensor] = None, chunk: int = 0,
                            sinks: Optional[torch.Tensor] = None) -> None:
    """Attention of every token of ``q`` [T, >= nh hd] (row stride free) over its request's cached keys.

    Token t belongs to row ``token_seq[t]`` of ``block_tables`` and sits at absolute position ``positions[t]``;
    it sees keys max(0, p - window + 1) .. p (window 0: all).  ``out`` is [T, nh hd].  ``slopes`` (float32 [nh]):
    head h's score of key j gains ``slopes[h] * (j - p)``.  ``chunk`` > 0: it sees only keys from (p // chunk) * chunk
    on.  ``sinks`` (float32 [nh]): the softmax denominator also holds exp(sinks[h]).
    """
    _dev(q, kcache, vcache, out, block_tables, token_seq, positions)
    t = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nh * hd, "q: bad shape")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[0] == t and out.shape[1] >= nh * hd
          and out.dtype is q.dtype, "out: bad shape")
    pages = kcache.shape[0]
    _need(kcache.is_contiguous() and vcache.is_contiguous() and tuple(kcache.shape) == (pages, nkv, page_size * hd)
          and tuple(vcache.shape) == (pages, nkv, page_size * hd) and kcache.dtype is vcache.dtype,
          "cache tensors must be [pages, nkv, page_size * hd] tiles")
    _need(block_tables.dim() == 2 and block_tables.dtype is torch.int32 and block_tables.is_contiguous(),
          "block_tables must be contiguous int32 [requests, blocks]")
    _i32(token_seq, "token_seq", t)
    _i32(positions, "positions", t)
    if slopes is not None:
        _dev(slopes)
        _need(slopes.dtype is torch.float32 and slopes.is_contiguous() and slopes.numel() == nh,
              "slopes must be contiguous float32, one per query head")
    if sinks is not None:
        _dev(sinks)
        _need(sinks.dtype is torch.float32 and sinks.is_contiguous() and sinks.numel() == nh,
              "sinks must be contiguous float32, one per query head")
    _need(chunk >= 0, "chunk must not be negative")
    _check(core().atoma_paged_attention_generic(
        _p(q), q.stride(0), _p(kcache), _p(vcache), _p(out), out.stride(0), _code(q, "q"), _code(kcache, "cache"),
        _p(block_tables), block_tables.shape[1], _p(token_seq), _p(positions), ctypes.c_float(scale), int(window),
        page_size, t, nh, nkv, hd, _p(slopes), int(chunk), _p(sinks), _stream()), "paged_attention_generic")


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def swiglu(gu: torch.Tensor, out: Optional[torch.Tensor] = None, block: int = 0, act: str = "silu") -> torch.Tensor:
    """out[t, i] = act(gate[t, i]) * up[t, i] for gu [T, 2 I]; ``act``: "silu", or "gelu_tanh" (gelu's tanh form).

    ``block`` 0: gate is the first half of a row and up the second; 16: blocks of 16 gate values followed by
    their 16 up values (the order of the fused gate-up product's weight rows).
    """
    _dev(gu)
    _need(gu.dim() == 2 and gu.is_contiguous() and gu.shape[1] % 2 == 0, "swiglu input must be contiguous [T, 2 I]")
    t, inter = gu.shape[0], gu.shape[1] // 2
    if out is None:
        out = torch.empty((t, inter), dtype=gu.dtype, device=gu.device)
    _need(out.is_contiguous() and tuple(out.shape) == (t, inter) and out.dtype is gu.dtype, "swiglu: bad out")
    _check(core().atoma_swiglu(_p(gu), _p(out), _code(gu, "swiglu input"), t, inter, int(block),
                               GATE_ACTIVATIONS[act], _stream()), "swiglu")
    return out


def gemm_generic(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, out: Optional[torch.Tensor] = None,
                 ) -> torch.Tensor:
    """a [M, K] times w [N, K] transposed, in true float32 arithmetic; any sizes."""
    _dev(a, w)
    _need(a.dim() == 2 and w.dim() == 2 and a.stride(1) == 1 and w.stride(1) == 1 and a.shape[1] == w.shape[1],
          f"gemm: a {tuple(a.shape)} and w {tuple(w.shape)} do not fit")
    m, k = a.shape
    n = w.shape[0]
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=a.device)
    _need(out.dim() == 2 and out.stride(1) == 1 and tuple(out.shape) == (m, n) and out.dtype is out_dtype,
          "gemm: bad out")
    _check(core().atoma_gemm_generic(_p(a), _code(a, "a"), _p(w), _code(w, "w"), _p(out), _code(out, "out"), m, n, k,
                                     a.stride(0) if m > 1 else k, w.stride(0) if n > 1 else k,
                                     out.stride(0) if m > 1 else n, _stream()), "gemm_generic")
    return out


# ------------------------------------------------------------------------------------------------------------
# mechanisms that only some architectures have: each module is compiled when a model first uses it

_modules = {}


def _module(name: str):
    lib = _modules.get(name)
    if lib is None:
        lib = _modules[name] = load_hip_module(name)
    return lib


def _f32(t: torch.Tensor, what: str, n: Optional[int] = None):
    _need(t.dtype is torch.float32 and t.is_contiguous(), f"{what} must be a contiguous float32 tensor")
    if n is not None:
        _need(t.numel() == n, f"{what} has {t.numel()} entries, {n} are needed")


def _term(delta: torch.Tensor, t: int, width: int):
    """(pointer, dtype code, planes, plane stride) of a delta [T, W] or of planes [S, T, W]."""
    _need(delta.is_contiguous() and tuple(delta.shape[-2:]) == (t, width) and delta.dim() in (2, 3),
          "a term must be contiguous [T, W] or [planes, T, W] and match resid")
    planes = delta.shape[0] if delta.dim() == 3 else 1
    return _p(delta), _code(delta, "term"), planes, ctypes.c_size_t(t * width)


def add_normed(resid: torch.Tensor, terms, w_post: Optional[torch.Tensor], eps_post: float,
               w_next: Optional[torch.Tensor] = None, eps_next: float = 0.0,
               out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """resid += rmsnorm(sum_i scale_i * term_i) * w_post (float32, in place); with ``w_next`` also returns
    rmsnorm(resid) * w_next in ``out_dtype``.  ``terms``: one or two (tensor, scale) pairs, each tensor [T, W] or
    planes [S, T, W] (summed), float32 or bfloat16.  Norm weights are float32.  Without ``w_post`` the sum joins the
    stream as it is: resid += sum_i scale_i * term_i."""
    _need(resid.dtype is torch.float32 and resid.dim() == 2 and resid.is_contiguous(), "resid must be float32 [T, W]")
    t, width = resid.shape
    _need(1 <= len(terms) <= 2, "one or two terms")
    _need(width <= 16000, "rows of more than 16,000 columns do not fit the kernel's row buffer")
    _dev(resid, w_post, w_next, *[d for d, _ in terms])
    if w_post is not None:
        _f32(w_post, "norm weight", width)
    out = None
    if w_next is not None:
        _f32(w_next, "norm weight", width)
        out = torch.empty((t, width), dtype=out_dtype, device=resid.device)
    a = _term(terms[0][0], t, width)
    b = _term(terms[1][0], t, width) if len(terms) > 1 else (_p(None), F32, 0, ctypes.c_size_t(0))
    _check(_module("layer_norms").atoma_add_normed(
        _p(resid), *a, ctypes.c_float(terms[0][1]), *b, ctypes.c_float(terms[1][1] if len(terms) > 1 else 0.0),
        _p(w_post), ctypes.c_float(eps_post), _p(w_next), ctypes.c_float(eps_next), _p(out),
        _code(out, "out") if out is not None else F32, t, width, _stream()), "add_normed")
    return out


def set_rows(resid: torch.Tensor, y: torch.Tensor, bias: torch.Tensor) -> None:
    """resid[t] = y[t] + bias, all float32: the stream's rows replaced by a map of them."""
    _dev(resid, y, bias)
    _need(resid.dtype is torch.float32 and resid.dim() == 2 and resid.is_contiguous(), "resid must be float32 [T, W]")
    t, width = resid.shape
    _f32(y, "the new rows", t * width)
    _f32(bias, "the bias row", width)
    _check(_module("layer_norms").atoma_set_rows(_p(resid), _p(y), _p(bias), t, width, _stream()), "set_rows")


def pack_pair(a: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[a | b] row by row in ``out_dtype`` for two float32 streams [T, W]."""
    _dev(a, b)
    _need(a.dim() == 2 and a.shape == b.shape, "pack_pair: two streams of one shape")
    _f32(a, "stream")
    _f32(b, "stream")
    t, width = a.shape
    out = torch.empty((t, 2 * width), dtype=out_dtype, device=a.device)
    _check(_module("layer_norms").atoma_pack_pair(_p(a), _p(b), _p(out), _code(out, "out"), t, width, _stream()),
           "pack_pair")
    return out


def qk_norm_rope(qk: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, rot_dim: int, wq: torch.Tensor,
                 wk: torch.Tensor, eps: float, q_out: torch.Tensor, kcache: Optional[torch.Tensor],
                 vcache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor], page_size: int, nh: int,
                 nkv: int, hd: int, hd_out: Optional[int] = None) -> None:
    """From qk float32 [T, >= (nh + nkv) hd]: q and k normed over their whole projections (weights wq [nh hd],
    wk [nkv hd]), the first ``rot_dim`` columns of every head rotated in neighbouring pairs by position *
    inv_freq[i]; q to ``q_out`` [T, nh hd], k into ``kcache`` tiles at ``slot_mapping``; ``vcache`` (optional)
    receives the k projection as it came.  ``hd_out`` > hd: heads leave ``hd_out`` wide, zeros beyond hd, in
    ``q_out`` [T, nh hd_out] and in the tiles."""
    hd_out = hd if hd_out is None else int(hd_out)
    _dev(qk, positions, inv_freq, wq, wk, q_out, kcache, vcache, slot_mapping)
    t = qk.shape[0]
    _need(qk.dtype is torch.float32 and qk.dim() == 2 and qk.stride(1) == 1 and qk.shape[1] >= (nh + nkv) * hd,
          "qk must be float32 [T, >= (nh + nkv) hd]")
    _i32(positions, "positions", t)
    _f32(inv_freq, "inv_freq", rot_dim // 2)
    _f32(wq, "q norm weight", nh * hd)
    _f32(wk, "k norm weight", nkv * hd)
    _need(hd_out >= hd and q_out.dim() == 2 and q_out.stride(1) == 1 and q_out.shape[0] == t
          and q_out.shape[1] >= nh * hd_out, "q_out must be [T, nh hd_out]")
    cache_code = _code(q_out, "q_out")
    if kcache is not None:
        _need(slot_mapping is not None, "a cache write needs slots")
        _i32(slot_mapping, "slot_mapping", t)
        pages = kcache.shape[0]
        _need(kcache.is_contiguous() and tuple(kcache.shape) == (pages, nkv, page_size * hd_out), "key tiles: bad shape")
        cache_code = _code(kcache, "cache")
        if vcache is not None:
            _need(vcache.is_contiguous() and tuple(vcache.shape) == tuple(kcache.shape)
                  and vcache.dtype is kcache.dtype, "value tiles must match the key tiles")
    else:
        _need(vcache is None, "values without keys")
    _check(_module("layer_norms").atoma_qk_norm_rope(
        _p(qk), qk.stride(0), _p(positions), _p(inv_freq), int(rot_dim), _p(wq), _p(wk), ctypes.c_float(eps),
        _p(q_out), q_out.stride(0), _code(q_out, "q_out"), _p(kcache), _p(vcache), cache_code, _p(slot_mapping),
        int(page_size), t, nh, nkv, hd, hd_out, _stream()), "qk_norm_rope")


def delta_prepare(proj: torch.Tensor, offsets, heads: int, kv_heads: int, dim: int, vdim: int, taps: int,
                  token_seq: torch.Tensor, q_start: torch.Tensor, state_slots: torch.Tensor, state: torch.Tensor,
                  taps_w: torch.Tensor, dt_pre: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor):
    """The inputs of the gated delta rule for every token (see delta_rule.hip): (q, k, v, beta, decay, k . q), all float32,
    from ``proj`` float32 [T, ld] whose columns ``offsets`` = (q, k, v, b) name; the convolution's state rows of each
    entry's request are read and then replaced."""
    _dev(proj, token_seq, q_start, state_slots, state, taps_w, dt_pre, dt_bias, a_log)
    t = proj.shape[0]
    s = state_slots.numel()
    nqk, nv, nd = kv_heads * dim, heads * vdim, heads * dim
    channels = 2 * nqk + nv
    off_q, off_k, off_v, off_b = (int(o) for o in offsets)
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1, "proj must be float32 [T, ld]")
    _need(max(off_q + nqk, off_k + nqk, off_v + nv, off_b + heads) <= proj.shape[1] and min(offsets) >= 0,
          "the projections' columns do not fit proj")
    _i32(token_seq, "token_seq", t)
    _i32(q_start, "q_start", s + 1)
    _i32(state_slots, "state_slots", s)
    _need(state.dtype is torch.float32 and state.dim() == 2 and state.is_contiguous()
          and state.shape[1] == (taps - 1) * channels + heads * vdim * dim, "state: bad shape")
    _f32(taps_w, "taps", channels * taps)
    _need(dt_pre.dtype is torch.float32 and dt_pre.stride(1) == 1 and tuple(dt_pre.shape) == (t, nd), "dt_pre: bad shape")
    _f32(dt_bias, "dt_bias", nd)
    _f32(a_log, "A_log", heads)
    dev = proj.device
    qn = torch.empty((t, nqk), dtype=torch.float32, device=dev)
    kn = torch.empty((t, nqk), dtype=torch.float32, device=dev)
    vn = torch.empty((t, nv), dtype=torch.float32, device=dev)
    beta = torch.empty((t, heads), dtype=torch.float32, device=dev)
    decay = torch.empty((t, nd), dtype=torch.float32, device=dev)
    kq = torch.empty((t, kv_heads), dtype=torch.float32, device=dev)
    _check(_module("delta_rule").atoma_delta_prepare(
        _p(proj), proj.stride(0), off_q, off_k, off_v, off_b, heads, kv_heads, dim, vdim, taps, _p(token_seq),
        _p(q_start), _p(state_slots), _p(state), ctypes.c_size_t(state.stride(0)), _p(taps_w), _p(dt_pre),
        dt_pre.stride(0) if t > 1 else nd, _p(dt_bias),
        _p(a_log), _p(qn), _p(kn), _p(vn), _p(beta), _p(decay), _p(kq), t, s, _stream()), "delta_prepare")
    return qn, kn, vn, beta, decay, kq


LOWRANK_UP_MAX_TOKENS = 32      # beyond, the general product reads a tile of the weight once for 64 tokens


def lowrank_up(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x float32 [T, K] (row stride free) times w [N, K] transposed, float32 out, for few tokens and a small K: the
    second half of a low-rank map (float32 multiply-adds in ascending order of k, as the general product's)."""
    _dev(x, w)
    t, k = x.shape
    n = w.shape[0]
    _need(x.dtype is torch.float32 and x.stride(1) == 1 and w.dim() == 2 and w.is_contiguous() and w.shape[1] == k,
          "lowrank_up: operands do not fit")
    out = torch.empty((t, n), dtype=torch.float32, device=x.device)
    _check(_module("delta_rule").atoma_lowrank_up(_p(x), x.stride(0) if t > 1 else k, _p(w), _code(w, "w"), _p(out), n,
                                                  t, n, k, _stream()), "lowrank_up")
    return out


def delta_scan(qn, kn, vn, beta, decay, kq, heads: int, kv_heads: int, dim: int, vdim: int, taps: int,
               q_start: torch.Tensor, state_slots: torch.Tensor, state: torch.Tensor) -> torch.Tensor:
    """The recurrence over every entry's tokens, from and into the requests' state rows; returns o float32 [T, heads vdim]."""
    _dev(qn, kn, vn, beta, decay, kq, q_start, state_slots, state)
    t, s = qn.shape[0], state_slots.numel()
    nqk, nv, nd = kv_heads * dim, heads * vdim, heads * dim
    for x, n, what in ((qn, nqk, "q"), (kn, nqk, "k"), (vn, nv, "v"), (beta, heads, "beta"), (decay, nd, "decay"),
                       (kq, kv_heads, "k . q")):
        _need(x.dtype is torch.float32 and x.is_contiguous() and tuple(x.shape) == (t, n), f"{what}: bad shape")
    _i32(q_start, "q_start", s + 1)
    _i32(state_slots, "state_slots", s)
    _need(state.dtype is torch.float32 and state.dim() == 2 and state.is_contiguous()
          and state.shape[1] == (taps - 1) * (2 * nqk + nv) + heads * vdim * dim, "state: bad shape")
    o = torch.empty((t, nv), dtype=torch.float32, device=qn.device)
    _check(_module("delta_rule").atoma_delta_scan(
        _p(qn), _p(kn), _p(vn), _p(beta), _p(decay), _p(kq), heads, kv_heads, dim, vdim, taps, _p(q_start), _p(state_slots),
        _p(state), ctypes.c_size_t(state.stride(0)), s, _p(o), _stream()), "delta_scan")
    return o


def delta_out(o: torch.Tensor, gate_pre: torch.Tensor, w: torch.Tensor, eps: float, heads: int, vdim: int,
              out_dtype: torch.dtype) -> torch.Tensor:
    """o / sqrt(mean over a head's columns of o^2 + eps) * w * sigmoid(gate_pre), in ``out_dtype``."""
    _dev(o, gate_pre, w)
    t = o.shape[0]
    _need(o.dtype is torch.float32 and o.is_contiguous() and tuple(o.shape) == (t, heads * vdim), "o: bad shape")
    _need(gate_pre.dtype is torch.float32 and gate_pre.stride(1) == 1 and tuple(gate_pre.shape) == (t, heads * vdim),
          "gate: bad shape")
    _f32(w, "norm weight", vdim)
    out = torch.empty((t, heads * vdim), dtype=out_dtype, device=o.device)
    _check(_module("delta_rule").atoma_delta_out(_p(o), _p(gate_pre), gate_pre.stride(0) if t > 1 else heads * vdim,
                                                 _p(w), ctypes.c_float(eps), _p(out),
                                                 _code(out, "out"), t, heads, vdim, _stream()), "delta_out")
    return out


# ---- a state-space recurrence with a scalar decay per head (state_space.hip) ----------------------------------------

def _ssd_state_ok(state, heads, groups, vdim, n, taps):
    channels = heads * vdim + 2 * groups * n
    _need(state.dtype is torch.float32 and state.dim() == 2 and state.is_contiguous()
          and state.shape[1] == (taps - 1) * channels + heads * vdim * n, "state: bad shape")
    _need(0 < n <= 256 and 1 <= taps <= 64 and heads % groups == 0, "state sizes up to 256 and up to 64 taps")
    return channels


def ssd_prepare(proj: torch.Tensor, offsets, heads: int, groups: int, vdim: int, n: int, taps: int,
                token_seq: torch.Tensor, q_start: torch.Tensor, state_slots: torch.Tensor, state: torch.Tensor,
                taps_w: torch.Tensor, conv_bias: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor):
    """The inputs of the recurrence for every token: (xbc [T, channels] after convolution, bias and SiLU; dt [T, heads]
    = softplus(raw + dt_bias); decay [T, heads] = exp(-exp(A_log) dt)), all float32, from ``proj`` float32 [T, ld]
    whose columns ``offsets`` = (z, first convolved channel, dt) name."""
    _dev(proj, token_seq, q_start, state_slots, state, taps_w, conv_bias, dt_bias, a_log)
    t, s = proj.shape[0], state_slots.numel()
    channels = _ssd_state_ok(state, heads, groups, vdim, n, taps)
    off_z, off_x, off_dt = (int(o) for o in offsets)
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1, "proj must be float32 [T, ld]")
    _need(min(off_z, off_x, off_dt) >= 0 and max(off_z + heads * vdim, off_x + channels, off_dt + heads) <= proj.shape[1],
          "the projections' columns do not fit proj")
    _i32(token_seq, "token_seq", t)
    _i32(q_start, "q_start", s + 1)
    _i32(state_slots, "state_slots", s)
    _f32(taps_w, "taps", channels * taps)
    _f32(conv_bias, "the convolution's bias", channels)
    _f32(dt_bias, "dt_bias", heads)
    _f32(a_log, "A_log", heads)
    dev = proj.device
    xbc = torch.empty((t, channels), dtype=torch.float32, device=dev)
    dt = torch.empty((t, heads), dtype=torch.float32, device=dev)
    decay = torch.empty((t, heads), dtype=torch.float32, device=dev)
    _check(_module("state_space").atoma_ssd_prepare(
        _p(proj), proj.stride(0), off_z, off_x, off_dt, heads, groups, vdim, n, taps, _p(token_seq), _p(q_start),
        _p(state_slots), _p(state), ctypes.c_size_t(state.stride(0)), _p(taps_w), _p(conv_bias), _p(dt_bias), _p(a_log),
        _p(xbc), _p(dt), _p(decay), t, _stream()), "ssd_prepare")
    return xbc, dt, decay


def ssd_conv_state(proj: torch.Tensor, off_x: int, heads: int, groups: int, vdim: int, n: int, taps: int,
                   q_start: torch.Tensor, state_slots: torch.Tensor, state: torch.Tensor) -> None:
    """The last ``taps - 1`` inputs of the convolution of every entry into its request's state row (an entry shorter
    than that shifts the old rows)."""
    _dev(proj, q_start, state_slots, state)
    s = state_slots.numel()
    channels = _ssd_state_ok(state, heads, groups, vdim, n, taps)
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and 0 <= off_x
          and off_x + channels <= proj.shape[1], "proj must be float32 [T, ld] and hold the channels")
    _i32(q_start, "q_start", s + 1)
    _i32(state_slots, "state_slots", s)
    _check(_module("state_space").atoma_ssd_conv_state(
        _p(proj), proj.stride(0), int(off_x), heads, groups, vdim, n, taps, _p(q_start), _p(state_slots), _p(state),
        ctypes.c_size_t(state.stride(0)), s, _stream()), "ssd_conv_state")


SSD_CHUNK_MIN_TOKENS = 16      # entries of at least this many tokens run 64 tokens at a time on the matrix cores


def ssd_scan(xbc: torch.Tensor, dt: torch.Tensor, decay: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor,
             heads: int, groups: int, vdim: int, n: int, taps: int, q_start: torch.Tensor,
             state_slots: torch.Tensor, state: torch.Tensor, counts=None) -> torch.Tensor:
    """The recurrence over every entry's tokens, from and into the requests' state rows; returns y float32
    [T, heads vdim] = S^T C + D x.  ``counts``: the entries' numbers of tokens on the host; with them, entries of
    ``SSD_CHUNK_MIN_TOKENS`` tokens or more (and a state of at most 128) are worked 64 tokens at a time by float32
    MFMAs, the others token by token.  Which of the two an entry gets depends on its own length alone."""
    _dev(xbc, dt, decay, a_log, d_skip, q_start, state_slots, state)
    t, s = xbc.shape[0], state_slots.numel()
    channels = _ssd_state_ok(state, heads, groups, vdim, n, taps)
    _need(xbc.dtype is torch.float32 and xbc.is_contiguous() and tuple(xbc.shape) == (t, channels), "xbc: bad shape")
    for x, what in ((dt, "dt"), (decay, "decay")):
        _need(x.dtype is torch.float32 and x.is_contiguous() and tuple(x.shape) == (t, heads), f"{what}: bad shape")
    _f32(d_skip, "D", heads)
    _f32(a_log, "A_log", heads)
    _i32(q_start, "q_start", s + 1)
    _i32(state_slots, "state_slots", s)
    y = torch.empty((t, heads * vdim), dtype=torch.float32, device=xbc.device)
    lib = _module("state_space")
    longest = shortest = 0
    if counts is not None and len(counts) and n <= lib.atoma_ssd_chunk_max_state():
        _need(len(counts) == s, "one count per entry")
        longest, shortest = int(max(counts)), int(min(counts))
    below = 1 << 30
    if longest >= SSD_CHUNK_MIN_TOKENS:
        below = SSD_CHUNK_MIN_TOKENS
        max_chunks = -(-longest // 64)
        lib.atoma_ssd_chunk_scratch_floats.restype = ctypes.c_size_t
        scores = torch.empty((lib.atoma_ssd_chunk_scratch_floats(s, max_chunks, groups),), dtype=torch.float32,
                             device=xbc.device)
        _check(lib.atoma_ssd_chunk(
            _p(xbc), _p(dt), _p(a_log), _p(d_skip), heads, groups, vdim, n, taps, _p(q_start), _p(state_slots), _p(state),
            ctypes.c_size_t(state.stride(0)), _p(y), s, below, _p(scores), max_chunks, _stream()), "ssd_chunk")
    if shortest < below:
        _check(lib.atoma_ssd_scan(
            _p(xbc), _p(dt), _p(decay), _p(d_skip), heads, groups, vdim, n, taps, _p(q_start), _p(state_slots), _p(state),
            ctypes.c_size_t(state.stride(0)), _p(y), s, below, _stream()), "ssd_scan")
    return y


def ssd_out(y: torch.Tensor, proj: torch.Tensor, off_z: int, w: torch.Tensor, eps: float, norm_groups: int,
            out_dtype: torch.dtype) -> torch.Tensor:
    """u = y * silu(z) with z the columns of ``proj`` from ``off_z`` on; u divided by the root mean square of each of
    its ``norm_groups`` equal parts, times w, in ``out_dtype``."""
    _dev(y, proj, w)
    t, inner = y.shape
    _need(y.dtype is torch.float32 and y.is_contiguous(), "y: bad shape")
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[0] == t
          and 0 <= off_z and off_z + inner <= proj.shape[1], "proj must be float32 [T, ld] and hold z")
    _need(norm_groups > 0 and inner % norm_groups == 0, "the norm's groups must divide the row")
    _f32(w, "norm weight", inner)
    out = torch.empty((t, inner), dtype=out_dtype, device=y.device)
    _check(_module("state_space").atoma_ssd_out(_p(y), _p(proj), proj.stride(0), int(off_z), _p(w), ctypes.c_float(eps),
                                                inner, int(norm_groups), _p(out), _code(out, "out"), t, _stream()),
           "ssd_out")
    return out


# ---- attention over one cached latent vector per token (latent.hip) ---------------------------------------------------

def latent_prepare(proj: torch.Tensor, offsets, heads: int, dim: int, rank: int, rank_p: int, w_norm: torch.Tensor,
                   eps: float, kcache: torch.Tensor, vcache: torch.Tensor, slot_mapping: torch.Tensor, page_size: int,
                   act_dtype: torch.dtype):
    """(q [T, heads dim] in ``act_dtype``, gate float32 [T, heads] = sigmoid) from ``proj`` float32 [T, ld] whose
    columns ``offsets`` = (q, down projection, gates) name; the normed down projection (rank numbers, zeros up to
    ``rank_p``) goes into both tiles of the token's cache slot."""
    _dev(proj, w_norm, kcache, vcache, slot_mapping)
    t = proj.shape[0]
    off_q, off_c, off_g = (int(o) for o in offsets)
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1, "proj must be float32 [T, ld]")
    _need(min(off_q, off_c, off_g) >= 0 and max(off_q + heads * dim, off_c + rank, off_g + heads) <= proj.shape[1],
          "the projections' columns do not fit proj")
    _f32(w_norm, "norm weight", rank)
    _i32(slot_mapping, "slot_mapping", t)
    pages = kcache.shape[0]
    _need(kcache.is_contiguous() and vcache.is_contiguous() and tuple(kcache.shape) == (pages, 1, page_size * rank_p)
          and tuple(vcache.shape) == (pages, 1, page_size * rank_p) and kcache.dtype is vcache.dtype
          and kcache.dtype is act_dtype, "cache tensors must be [pages, 1, page_size * rank] tiles of the activation dtype")
    q = torch.empty((t, heads * dim), dtype=act_dtype, device=proj.device)
    gate = torch.empty((t, heads), dtype=torch.float32, device=proj.device)
    _check(_module("latent").atoma_latent_prepare(
        _p(proj), proj.stride(0), off_q, off_c, off_g, heads * dim, rank, rank_p, heads, _p(w_norm), ctypes.c_float(eps),
        _p(kcache), _p(vcache), _code(kcache, "cache"), _p(slot_mapping), page_size, _p(q), _code(q, "q"), _p(gate), t,
        _stream()), "latent_prepare")
    return q, gate


def head_linear(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype, gate: Optional[torch.Tensor] = None,
                ) -> torch.Tensor:
    """Per head a product of its own: x [T, H K] (row stride free), w [H, N, K] -> [T, H N] in ``out_dtype``, float32
    sums; with ``gate`` float32 [T, H] every head's result is multiplied by its number, with ``gate`` [T, H N] every
    output by its own."""
    _dev(x, w, gate)
    _need(w.dim() == 3 and w.is_contiguous(), "head_linear: w must be contiguous [H, N, K]")
    h, n, k = w.shape
    t = x.shape[0]
    _need(x.dim() == 2 and x.stride(1) == 1 and x.shape[1] == h * k, "head_linear: x must be [T, H K]")
    gate_cols = 0
    if gate is not None:
        gate_cols = int(gate.numel() == t * h * n and n > 1)
        _f32(gate, "gate", t * h * n if gate_cols else t * h)
    out = torch.empty((t, h * n), dtype=out_dtype, device=x.device)
    _check(_module("latent").atoma_head_linear(_p(x), _code(x, "x"), x.stride(0) if t > 1 else h * k, _p(w), _code(w, "w"),
                                               _p(out), _code(out, "out"), h * n, _p(gate), gate_cols, t, h, k, n,
                                               _stream()), "head_linear")
    return out



def route_topk(logits: torch.Tensor, top: int, score: str = "sigmoid", correction: Optional[torch.Tensor] = None,
               scale: float = 1.0):
    """(ids int32 [T, top], weights float32 [T, top]).  Scores are sigmoid(logits) or ("softmax") the softmax of a
    row; the ``top`` experts with the largest score + ``correction`` [experts] are chosen and weighed by
    score * ``scale``."""
    _dev(logits, correction)
    _need(score in ("sigmoid", "softmax"), "route_topk: scores are 'sigmoid' or 'softmax'")
    if correction is not None:
        _f32(correction, "correction", logits.shape[1])
    _need(logits.dtype is torch.float32 and logits.dim() == 2 and logits.stride(1) == 1, "router logits: float32 [T, E]")
    t, e = logits.shape
    ids = torch.empty((t, top), dtype=torch.int32, device=logits.device)
    scores = torch.empty((t, top), dtype=torch.float32, device=logits.device)
    _check(_module("experts").atoma_route_topk(_p(logits), logits.stride(0), e, int(top), _p(ids), _p(scores), t,
                                               1 if score == "softmax" else 0, _p(correction), ctypes.c_float(scale),
                                               _stream()), "route_topk")
    return ids, scores


def route_group(ids: torch.Tensor, experts: int, tile_m: int = 64):
    """Slots (token, choice) ordered by expert: (perm int32 [slots], offsets int32 [experts + 1], tiles int32
    [max_tiles, 2] of (expert or -1, first place in perm)); a tile holds up to ``tile_m`` (64 or 128) places."""
    _dev(ids)
    _i32(ids, "ids")
    n = ids.numel()
    lib = _module("experts")
    max_tiles = int(lib.atoma_route_max_tiles(n, experts, int(tile_m)))
    perm = torch.empty(n, dtype=torch.int32, device=ids.device)
    offsets = torch.empty(experts + 1, dtype=torch.int32, device=ids.device)
    tiles = torch.empty((max_tiles, 2), dtype=torch.int32, device=ids.device)
    _check(lib.atoma_route_group(_p(ids), n, experts, _p(perm), _p(offsets), _p(tiles), max_tiles, int(tile_m),
                                 _stream()), "route_group")
    return perm, offsets, tiles


def expert_gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, perm, offsets, tiles, top: int, *,
                gather: bool, scale: Optional[torch.Tensor] = None, planes: bool = False, relu2: bool = False,
                out_scale: Optional[torch.Tensor] = None) -> None:
    """out[row(slot)] = (scale[slot] * a[src(slot)]) @ w[expert(slot)]^T in float32 arithmetic, for every slot.
    ``gather``: src is the slot's token (a [T, K]), else the slot (a [slots, K]).  ``planes``: out is [top, T, N]
    and choice c of token t goes to out[c, t], else out is [slots, N].  ``relu2``: the result's positive part squared;
    ``out_scale`` [slots] multiplies the result."""
    _dev(a, w, out, perm, offsets, tiles, scale, out_scale)
    if out_scale is not None:
        _f32(out_scale, "out_scale", perm.numel())
    n_slots = perm.numel()
    e, n, k = w.shape
    _need(w.is_contiguous() and a.dim() == 2 and a.stride(1) == 1 and a.shape[1] == k, "expert_gemm: a and w do not fit")
    _need(a.shape[0] * (top if gather else 1) == n_slots, "expert_gemm: rows of a do not fit the slots")
    _need(out.is_contiguous() and out.numel() == n_slots * n and out.shape[-1] == n, "expert_gemm: bad out")
    _need(offsets.numel() == e + 1 and tiles.dim() == 2 and tiles.shape[1] == 2, "expert_gemm: bad grouping")
    if scale is not None:
        _need(scale.dtype is torch.float32 and scale.is_contiguous() and scale.numel() == n_slots, "expert_gemm: bad scale")
    _check(_module("experts").atoma_expert_gemm(
        _p(a), _code(a, "a"), a.stride(0) if a.shape[0] > 1 else k, top if gather else 1, _p(scale), _p(w),
        _code(w, "w"), _p(out), _code(out, "out"), n, n, k, _p(perm), _p(offsets), _p(tiles), tiles.shape[0], int(top),
        n_slots // top if planes else 0, 2 if relu2 else 0, _p(out_scale), _stream()), "expert_gemm")


def gather_scale(x: torch.Tensor, scores: Optional[torch.Tensor], perm: torch.Tensor, top: int) -> torch.Tensor:
    """xs[place] = bfloat16(scores[slot] * x[slot // top]) for slot = perm[place]: the experts' inputs in their order
    (without ``scores``: the inputs as they are)."""
    _dev(x, scores, perm)
    n, k = perm.numel(), x.shape[1]
    _need(x.dtype is torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1 and x.shape[0] * top == n, "gather_scale: bad x")
    if scores is not None:
        _f32(scores, "scores", n)
    _i32(perm, "perm", n)
    xs = torch.empty((n, k), dtype=torch.bfloat16, device=x.device)
    _check(_module("experts").atoma_gather_scale(_p(x), x.stride(0) if x.shape[0] > 1 else k, _p(scores), _p(perm),
                                                 _p(xs), k, int(top), n, _stream()), "gather_scale")
    return xs


def expert_gemm_mfma_ok(n: int, k: int) -> bool:
    return k % 32 == 0 and n % 32 == 0


def expert_gemm_mfma(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, perm, offsets, tiles, top: int, *,
                     swiglu: bool = False, planes: bool = False, tile_m: int = 64, relu2: bool = False,
                     out_scale: Optional[torch.Tensor] = None) -> None:
    """The grouped product on the matrix cores: a bfloat16 [places, K] in the order of ``perm``, w bfloat16
    [experts, N, K].  ``swiglu``: w's rows in blocks of 16 gate rows and their 16 up rows, out bfloat16
    [places, N / 2] = silu(gate) * up; ``relu2``: out bfloat16 [places, N], the result's positive part squared; else out
    float32 [places, N] or, with ``planes``, [top, T, N] by slot, times ``out_scale`` [slots] where given.
    ``tile_m``: what ``route_group`` was told."""
    _dev(a, w, out, perm, offsets, tiles, out_scale)
    _need(not (swiglu and relu2), "expert_gemm_mfma: one activation")
    if out_scale is not None:
        _f32(out_scale, "out_scale", perm.numel())
    n_slots = perm.numel()
    e, n, k = w.shape
    _need(a.dtype is torch.bfloat16 and w.dtype is torch.bfloat16 and a.is_contiguous() and w.is_contiguous()
          and tuple(a.shape) == (n_slots, k) and expert_gemm_mfma_ok(n, k), "expert_gemm_mfma: operands do not fit")
    cols = n // 2 if swiglu else n
    _need(out.is_contiguous() and out.numel() == n_slots * cols and out.shape[-1] == cols
          and out.dtype is (torch.bfloat16 if swiglu or relu2 else torch.float32)
          and not ((swiglu or relu2) and (planes or out_scale is not None)), "expert_gemm_mfma: bad out")
    _need(offsets.numel() == e + 1 and tiles.dim() == 2 and tiles.shape[1] == 2, "expert_gemm_mfma: bad grouping")
    _check(_module("experts").atoma_expert_gemm_mfma(
        _p(a), _p(w), _p(out), cols, n, k, _p(perm), _p(offsets), _p(tiles), tiles.shape[0], int(top),
        n_slots // top if planes else 0, 1 if swiglu else 2 if relu2 else 0, int(tile_m), _p(out_scale), _stream()),
        "expert_gemm_mfma")


def relu2_gate(u: torch.Tensor, ff: int, off_gate: int, out_dtype: torch.dtype) -> torch.Tensor:
    """out[t, i] = relu(u[t, i])^2 * sigmoid(u[t, off_gate]) for i < ff (``off_gate`` < 0: no gate), u [T, >= ff]."""
    _dev(u)
    _need(u.dim() == 2 and u.stride(1) == 1 and u.shape[1] >= ff and off_gate < u.shape[1], "relu2_gate: bad input")
    t = u.shape[0]
    out = torch.empty((t, ff), dtype=out_dtype, device=u.device)
    _check(_module("experts").atoma_relu2_gate(_p(u), _code(u, "u"), u.stride(0) if t > 1 else u.shape[1], _p(out),
                                               _code(out, "out"), t, int(ff), int(off_gate), _stream()), "relu2_gate")
    return out


def depth_average(resid: torch.Tensor, terms, w_post: Optional[torch.Tensor], eps_post: float, results: torch.Tensor,
                  n: int, weights: torch.Tensor, w_next: Optional[torch.Tensor] = None, eps_next: float = 0.0,
                  out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """X = resid + rmsnorm(sum_i scale_i * term_i) * w_post is kept as results[n - 1]; resid becomes
    sum_(j < n) weights[j] * results[j] (float32); with ``w_next`` also returns rmsnorm(resid) * w_next in
    ``out_dtype``.  ``results``: float32 [>= n, T, W]; ``terms`` as for ``add_normed``."""
    _need(resid.dtype is torch.float32 and resid.dim() == 2 and resid.is_contiguous(), "resid must be float32 [T, W]")
    t, width = resid.shape
    _need(1 <= len(terms) <= 2, "one or two terms")
    _need(width <= 16000, "rows of more than 16,000 columns do not fit the kernel's row buffer")
    _dev(resid, w_post, w_next, results, weights, *[d for d, _ in terms])
    _need(results.dtype is torch.float32 and results.dim() == 3 and results.is_contiguous()
          and tuple(results.shape[1:]) == (t, width) and 1 <= n <= results.shape[0], "depth_average: bad results")
    _f32(weights, "depth weights", n)
    if w_post is not None:
        _f32(w_post, "norm weight", width)
    out = None
    if w_next is not None:
        _f32(w_next, "norm weight", width)
        out = torch.empty((t, width), dtype=out_dtype, device=resid.device)
    a = _term(terms[0][0], t, width)
    b = _term(terms[1][0], t, width) if len(terms) > 1 else (_p(None), F32, 0, ctypes.c_size_t(0))
    _check(_module("layer_norms").atoma_depth_average(
        _p(resid), *a, ctypes.c_float(terms[0][1]), *b, ctypes.c_float(terms[1][1] if len(terms) > 1 else 0.0),
        _p(w_post), ctypes.c_float(eps_post), _p(results), ctypes.c_size_t(t * width), int(n), _p(weights), _p(w_next),
        ctypes.c_float(eps_next), _p(out), _code(out, "out") if out is not None else F32, t, width, _stream()),
        "depth_average")
    return out


def diff_prepare(proj: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, rot_dim: int, q_out: torch.Tensor,
                 kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor],
                 page_size: int, heads: int, kv_heads: int, dim: int, vdim: int, hdo: int, offsets) -> torch.Tensor:
    """Differential attention's inputs from the fused projection [q | k | v | g] (see differential.hip): rotated
    queries to ``q_out`` [T, 2 heads, hdo], keys [k1 | k2 | 0] and values [v | 0] into their tiles, and the heads'
    gates, sigmoid applied, as float32 [T, heads] (returned).  ``offsets`` = (k, v, g) columns of ``proj``; without
    tiles ``proj`` needs q and g only."""
    _dev(proj, positions, inv_freq, q_out, kcache, vcache, slot_mapping)
    t = proj.shape[0]
    off_k, off_v, off_g = (int(o) for o in offsets)
    _need(proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= off_g + heads, "diff_prepare: bad projection")
    _need(2 * heads * dim <= min(off_g, off_k if kcache is not None else off_g), "diff_prepare: offsets overlap q")
    _i32(positions, "positions", t)
    _f32(inv_freq, "inv_freq", rot_dim // 2)
    _need(q_out.dim() == 2 and q_out.is_contiguous() and tuple(q_out.shape) == (t, 2 * heads * hdo), "diff_prepare: bad q_out")
    cache_code = _code(q_out, "q_out")
    if kcache is not None:
        _need(slot_mapping is not None and vcache is not None, "a cache write needs slots and both tiles")
        _i32(slot_mapping, "slot_mapping", t)
        _need(off_k + 2 * kv_heads * dim <= off_v and off_v + kv_heads * vdim <= off_g, "diff_prepare: offsets overlap")
        pages = kcache.shape[0]
        _need(kcache.is_contiguous() and tuple(kcache.shape) == (pages, kv_heads, page_size * hdo)
              and vcache.is_contiguous() and tuple(vcache.shape) == tuple(kcache.shape)
              and vcache.dtype is kcache.dtype, "diff_prepare: the tiles must be [pages, kv_heads, page_size * hdo]")
        cache_code = _code(kcache, "cache")
    gate = torch.empty((t, heads), dtype=torch.float32, device=proj.device)
    _check(_module("differential").atoma_diff_prepare(
        _p(proj), _code(proj, "proj"), proj.stride(0) if t > 1 else proj.shape[1], _p(positions), _p(inv_freq),
        int(rot_dim), _p(q_out), q_out.stride(0), _code(q_out, "q_out"), _p(kcache), _p(vcache), cache_code,
        _p(slot_mapping), int(page_size), _p(gate), t, heads, kv_heads, dim, vdim, hdo, off_k, off_v, off_g, _stream()),
        "diff_prepare")
    return gate


def diff_combine(att: torch.Tensor, gate: torch.Tensor, heads: int, vdim: int, hdo: int, lam: float, eps: float,
                 post: float, out_dtype: torch.dtype) -> torch.Tensor:
    """y[t, h] = (a1 - lam a2) / sqrt(mean((a1 - lam a2)^2) + eps) * post * gate[t, h] over the first ``vdim`` columns
    of the two maps' outputs att[t, 2h] and att[t, 2h + 1] ([T, 2 heads * hdo]); y [T, heads * vdim]."""
    _dev(att, gate)
    t = att.shape[0]
    _need(att.dim() == 2 and att.is_contiguous() and att.shape[1] == 2 * heads * hdo, "diff_combine: bad input")
    _f32(gate, "gate", t * heads)
    y = torch.empty((t, heads * vdim), dtype=out_dtype, device=att.device)
    _check(_module("differential").atoma_diff_combine(
        _p(att), _code(att, "att"), att.shape[1], _p(gate), _p(y), _code(y, "y"), heads * vdim, t, heads, vdim, hdo,
        ctypes.c_float(lam), ctypes.c_float(eps), ctypes.c_float(post), _stream()), "diff_combine")
    return y


MINGRU_STRETCH_MIN_TOKENS = 64      # entries of at least this many tokens are walked in stretches side by side


def mingru_plan(counts, width: int, compute_units: int = 256, min_length: int = 16):
    """The stretches of a step for ``mingru``: int32 [n][3] of (entry, first token, end) followed by [entries + 1] of
    each entry's first stretch; None when no entry is long enough to pay for it.  A function of the entries' lengths.
    ``min_length``: the shortest stretch (a recurrence whose walk over an entry's stretches costs two dependent loads
    a stretch asks for longer ones)."""
    import numpy as np
    counts = np.asarray(counts, dtype=np.int64)
    if counts.size == 0 or int(counts.max()) < MINGRU_STRETCH_MIN_TOKENS:
        return None
    # stretches long enough to amortise the second read of their tokens, short enough that the step's stretches
    # times the channels' workgroups give every compute unit a few workgroups
    blocks = -(-width // 256)
    total = int(counts.sum())
    length = max(int(min_length), min(256, (total * blocks) // (4 * compute_units)))
    rows, first, t0 = [], [0], 0
    for e, c in enumerate(counts.tolist()):
        for lo in range(0, c, length):
            rows.append((e, t0 + lo, t0 + min(lo + length, c)))
        first.append(len(rows))
        t0 += c
    if len(rows) > 65535:
        return None
    return np.concatenate([np.asarray(rows, dtype=np.int32).reshape(-1), np.asarray(first, dtype=np.int32)]), len(rows)


def mingru(proj: torch.Tensor, off_x: int, off_g: int, width: int, bz: torch.Tensor, bx: torch.Tensor,
           q_start: torch.Tensor, state_slots: torch.Tensor, state: torch.Tensor, out_dtype: torch.dtype,
           plan=None) -> torch.Tensor:
    """The minGRU recurrence over a step's entries (see mingru.hip): proj float32 [T, >= off_g + width] holds the
    columns of z (from 0), x and g; y [T, width] = S * silu(g) with each request's S [width] read from and written to
    its row of ``state``.  ``plan``: (int32 device tensor, stretches) from ``mingru_plan``, or None for the plain walk."""
    _dev(proj, bz, bx, q_start, state_slots, state)
    t = proj.shape[0]
    n_entries = state_slots.numel()
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[1] >= off_g + width
          and off_x >= width and off_g >= off_x + width, "mingru: bad projection")
    _f32(bz, "z bias", width)
    _f32(bx, "x bias", width)
    _i32(q_start, "q_start", n_entries + 1)
    _i32(state_slots, "state_slots")
    _need(state.dtype is torch.float32 and state.is_contiguous() and state.dim() == 2 and state.shape[1] == width,
          "mingru: the state must be float32 [slots, width]")
    y = torch.empty((t, width), dtype=out_dtype, device=proj.device)
    ld = proj.stride(0) if t > 1 else proj.shape[1]
    lib = _module("mingru")
    if plan is None or plan[1] == 0:
        _check(lib.atoma_mingru_scan(_p(proj), ld, _p(bz), _p(bx), _p(q_start), _p(state_slots), _p(state), _p(y),
                                     _code(y, "y"), width, n_entries, width, int(off_x), int(off_g), _stream()),
               "mingru_scan")
        return y
    arr, n_st = plan
    _i32(arr, "stretches", 3 * n_st + n_entries + 1)
    ab = torch.empty((n_st, 2, width), dtype=torch.float32, device=proj.device)
    first = ctypes.c_void_p(arr.data_ptr() + 12 * n_st)
    _check(lib.atoma_mingru_stretched(_p(proj), ld, _p(bz), _p(bx), _p(arr), int(n_st), first, _p(state_slots),
                                      _p(state), _p(ab), _p(y), _code(y, "y"), width, n_entries, width, int(off_x),
                                      int(off_g), _stream()), "mingru_stretched")
    return y


# -- a stream kept in several copies, and the embedding that starts it ------------------------------------------

MAX_STREAM_COPIES = 8


def _planes(y: torch.Tensor, t: int, width: int, what: str):
    _need(y.is_contiguous() and y.dim() in (2, 3) and tuple(y.shape[-2:]) == (t, width),
          f"{what} must be contiguous [T, W] or [planes, T, W]")
    return y.shape[0] if y.dim() == 3 else 1


def stream_step(x: torch.Tensor, update=None, read=None, rows: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
    """One pass over the copies x float32 [S, T, W] of the residual stream.

    ``update`` = (y, mix float32 [S, S] indexed [from, to], out float32 [S]): every copy becomes
    ``sum_s mix[s, t] x_s + out[t] y``, all from the old ones; y is [T, W] or float32 planes [P, T, W] (summed).
    ``read`` = (w_in float32 [S], norm weight float32 [W], eps): returns ``rmsnorm(sum_s w_in[s] x_s) * weight`` of the
    new copies in ``out_dtype``.  With ``rows`` (int32) only those rows are read and x is left as it was."""
    _need(x.dtype is torch.float32 and x.dim() == 3 and x.is_contiguous(), "the stream must be float32 [S, T, W]")
    s, t, width = x.shape
    _need(1 <= s <= MAX_STREAM_COPIES, f"1 to {MAX_STREAM_COPIES} copies of the stream")
    _need(update is not None or read is not None, "stream_step: nothing to do")
    y = mix = outw = inw = nw = h = None
    planes, eps = 0, 0.0
    if update is not None:
        y, mix, outw = update
        planes = _planes(y, t, width, "the sublayer's output")
        _f32(mix, "mix", s * s)
        _f32(outw, "out weights", s)
    if read is not None:
        inw, nw, eps = read
        _f32(inw, "in weights", s)
        _f32(nw, "norm weight", width)
        n = rows.numel() if rows is not None else t
        h = torch.empty((n, width), dtype=out_dtype, device=x.device)
    if rows is not None:
        _i32(rows, "rows")
        _need(read is not None, "rows are for reading")
    _dev(x, y, mix, outw, inw, nw, rows)
    _check(_module("streams").atoma_stream_step(
        _p(x), t, width, s, _p(y), _code(y, "y") if y is not None else F32, planes, ctypes.c_size_t(t * width),
        _p(mix), _p(outw), _p(inw), _p(nw), ctypes.c_float(eps), _p(h), _code(h, "out") if h is not None else F32,
        _p(rows), rows.numel() if rows is not None else 0, int(rows is None), _stream()), "stream_step")
    return h


def bigram_embed(tokens, positions, token_seq, q_start, state_slots, state: Optional[torch.Tensor],
                 table: torch.Tensor, pairs: Optional[torch.Tensor], buckets: int, mul_prev: int, mul_cur: int,
                 scale: float, copies: int) -> torch.Tensor:
    """x float32 [copies, T, W], every copy ``table[token] * scale + pairs[(prev * mul_prev + token * mul_cur) mod
    buckets]`` (row ``buckets`` of ``pairs`` at position 0; ``pairs`` None: the first term alone).  ``state`` int32
    [slots, 1] holds each request's last token between steps."""
    _dev(tokens, positions, token_seq, q_start, state_slots, state, table, pairs)
    t, s = tokens.numel(), state_slots.numel()
    _i32(tokens, "tokens")
    _i32(positions, "positions", t)
    _i32(token_seq, "token_seq", t)
    _i32(q_start, "q_start", s + 1)
    _i32(state_slots, "state_slots")
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [vocab, width]")
    width = table.shape[1]
    if pairs is not None:
        _need(pairs.is_contiguous() and tuple(pairs.shape) == (buckets + 1, width) and pairs.dtype is table.dtype,
              "the pair table must be [buckets + 1, width] of the embedding's dtype")
        _need(state is not None and state.dtype is torch.int32 and state.is_contiguous() and state.dim() == 2
              and state.shape[1] == 1, "the previous-token state must be int32 [slots, 1]")
    x = torch.empty((copies, t, width), dtype=torch.float32, device=table.device)
    _check(_module("streams").atoma_bigram_embed(
        _p(tokens), _p(positions), _p(token_seq), _p(q_start), _p(state_slots), _p(state), _p(table),
        _code(table, "embedding table"), table.shape[0], _p(pairs), int(buckets), ctypes.c_longlong(mul_prev),
        ctypes.c_longlong(mul_cur), ctypes.c_float(scale), _p(x), t, int(copies), width, _stream()), "bigram_embed")
    return x


def normed_branches(a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, eps: float, scale: float,
                    bias_a: Optional[torch.Tensor] = None, bias_b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [T, W]: ``scale * (rmsnorm(a + bias_a) * wa + rmsnorm(b + bias_b) * wb)``; a and b are [T, W] or
    float32 planes [P, T, W] (summed first)."""
    t, width = a.shape[-2:]
    pa, pb = _planes(a, t, width, "a branch"), _planes(b, t, width, "a branch")
    _dev(a, b, wa, wb, bias_a, bias_b)
    _f32(wa, "norm weight", width)
    _f32(wb, "norm weight", width)
    for bias in (bias_a, bias_b):
        if bias is not None:
            _f32(bias, "bias", width)
    y = torch.empty((t, width), dtype=torch.float32, device=a.device)
    _check(_module("streams").atoma_normed_branches(_p(a), _code(a, "a"), pa, _p(b), _code(b, "b"), pb, _p(bias_a),
                                                    _p(bias_b), _p(wa), _p(wb), ctypes.c_float(eps),
                                                    ctypes.c_float(scale), _p(y), t, width, _stream()),
           "normed_branches")
    return y


def dense_act(u: torch.Tensor, out_dtype: torch.dtype, act: str = "relu2") -> torch.Tensor:
    """act(u) for u [T, I] (float32 or bfloat16) in ``out_dtype``; ``act``: "relu2", the square of relu."""
    _dev(u)
    _need(act == "relu2", f"dense_act: unknown activation {act!r}")
    _need(u.dim() == 2 and u.stride(1) == 1, "dense_act: u must be [T, I]")
    t, inter = u.shape
    out = torch.empty((t, inter), dtype=out_dtype, device=u.device)
    _check(core().atoma_dense_act(_p(u), _code(u, "u"), u.stride(0) if t > 1 else inter, _p(out), _code(out, "out"), t,
                                  inter, 0, _stream()), "dense_act")
    return out


# -- gated attention kinds: the kernels between projections and attention ---------------------------------------

def _tiles_ok(kcache, vcache, nkv, page_size, hd):
    pages = kcache.shape[0]
    _need(kcache.is_contiguous() and vcache is not None and vcache.is_contiguous()
          and tuple(kcache.shape) == (pages, nkv, page_size * hd) and tuple(vcache.shape) == tuple(kcache.shape)
          and kcache.dtype is vcache.dtype, "cache tensors must be [pages, kv_heads, page_size * head] tiles of one dtype")


def tied_rope_prepare(proj: torch.Tensor, offsets, bq, bk, positions, freq: torch.Tensor, rot: int, interleaved: bool,
                      mag: float, kcache, vcache, slot_mapping, page_size: int, nh: int, nkv: int, hd: int,
                      hd_out: int, act_dtype: torch.dtype):
    """(q [T, nh hd_out] in ``act_dtype``, gate float32 [T, nh hd] = sigmoid) from ``proj`` float32 [T, ld] whose
    columns ``offsets`` = (q, k, g) name; k with its bias goes into the value tiles as it is and rotated into the key
    tiles (see gated_attention.hip)."""
    _dev(proj, bq, bk, positions, freq, kcache, vcache, slot_mapping)
    t = proj.shape[0]
    off_q, off_k, off_g = (int(o) for o in offsets)
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1, "proj must be float32 [T, ld]")
    _need(min(off_q, off_k, off_g) >= 0 and max(off_q + nh * hd, off_k + nkv * hd, off_g + nh * hd) <= proj.shape[1],
          "the projections' columns do not fit proj")
    if bq is not None:
        _f32(bq, "q bias", nh * hd)
    if bk is not None:
        _f32(bk, "k bias", nkv * hd)
    _i32(positions, "positions", t)
    _i32(slot_mapping, "slot_mapping", t)
    _f32(freq, "frequencies", rot // 2)
    _tiles_ok(kcache, vcache, nkv, page_size, hd_out)
    _need(kcache.dtype is act_dtype, "the cache must be of the activation dtype")
    q = torch.empty((t, nh * hd_out), dtype=act_dtype, device=proj.device)
    gate = torch.empty((t, nh * hd), dtype=torch.float32, device=proj.device)
    _check(_module("gated_attention").atoma_tied_rope_prepare(
        _p(proj), proj.stride(0), off_q, off_k, off_g, _p(bq), _p(bk), _p(positions), _p(freq), int(rot),
        int(bool(interleaved)), ctypes.c_float(mag), _p(q), _code(q, "q"), _p(kcache), _p(vcache),
        _code(kcache, "cache"), _p(slot_mapping), int(page_size), _p(gate), t, nh, nkv, hd, hd_out, _stream()),
        "tied_rope_prepare")
    return q, gate


def latent_rope_prepare(proj: torch.Tensor, offsets, q_rank: int, rank: int, rd: int, rank_p: int, n_gate: int,
                        wq: torch.Tensor, wc: torch.Tensor, eps: float, positions, freq: torch.Tensor, rot: int,
                        kcache, vcache, slot_mapping, page_size: int, act_dtype: torch.dtype):
    """(cq [T, q_rank] in ``act_dtype``, gate float32 [T, n_gate] = sigmoid) from ``proj`` float32 [T, ld] whose columns
    ``offsets`` = (query latent, key/value latent followed by the rotated key part, gates) name; the cache tiles
    receive [c | rotated part | 0] as the key and [c | 0] as the value, ``rank_p`` columns each."""
    _dev(proj, wq, wc, positions, freq, kcache, vcache, slot_mapping)
    t = proj.shape[0]
    off_dq, off_c, off_g = (int(o) for o in offsets)
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1, "proj must be float32 [T, ld]")
    _need(min(off_dq, off_c, off_g) >= 0 and max(off_dq + q_rank, off_c + rank + rd, off_g + n_gate) <= proj.shape[1],
          "the projections' columns do not fit proj")
    _f32(wq, "norm weight", q_rank)
    _f32(wc, "norm weight", rank)
    _i32(positions, "positions", t)
    _i32(slot_mapping, "slot_mapping", t)
    _f32(freq, "frequencies", rot // 2)
    _tiles_ok(kcache, vcache, 1, page_size, rank_p)
    _need(kcache.dtype is act_dtype, "the cache must be of the activation dtype")
    cq = torch.empty((t, q_rank), dtype=act_dtype, device=proj.device)
    gate = torch.empty((t, n_gate), dtype=torch.float32, device=proj.device)
    _check(_module("gated_attention").atoma_latent_rope_prepare(
        _p(proj), proj.stride(0), off_dq, off_c, off_g, q_rank, rank, rd, rank_p, n_gate, _p(wq), _p(wc),
        ctypes.c_float(eps), _p(positions), _p(freq), int(rot), _p(cq), _code(cq, "cq"), _p(kcache), _p(vcache),
        _code(kcache, "cache"), _p(slot_mapping), int(page_size), _p(gate), t, _stream()), "latent_rope_prepare")
    return cq, gate


def latent_q_rope(q: torch.Tensor, positions, freq: torch.Tensor, rot: int, heads: int, dim: int, rd: int,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """q float32 [T, heads (dim + rd)] in ``out_dtype`` with the first ``rot`` of every head's last ``rd`` columns
    rotated in neighbouring pairs."""
    _dev(q, positions, freq)
    t = q.shape[0]
    _need(q.dtype is torch.float32 and q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= heads * (dim + rd),
          "q must be float32 [T, heads (dim + rd)]")
    _i32(positions, "positions", t)
    _f32(freq, "frequencies", rot // 2)
    out = torch.empty((t, heads * (dim + rd)), dtype=out_dtype, device=q.device)
    _check(_module("gated_attention").atoma_latent_q_rope(_p(q), q.stride(0), _p(positions), _p(freq), int(rot), _p(out),
                                                          _code(out, "out"), t, heads, dim, rd, _stream()),
           "latent_q_rope")
    return out


def gate_mul(att: torch.Tensor, gate: torch.Tensor, heads: int, vd: int, hd_out: int) -> torch.Tensor:
    """[T, heads vd]: the first ``vd`` of every head's ``hd_out`` columns of ``att`` times ``gate`` float32 [T, heads vd]."""
    _dev(att, gate)
    t = att.shape[0]
    _need(att.is_contiguous() and tuple(att.shape) == (t, heads * hd_out), "att must be contiguous [T, heads hd_out]")
    _f32(gate, "gate", t * heads * vd)
    y = torch.empty((t, heads * vd), dtype=att.dtype, device=att.device)
    _check(_module("gated_attention").atoma_gate_mul(_p(att), _p(gate), _p(y), _code(att, "att"), t, heads, vd, hd_out,
                                                     _stream()), "gate_mul")
    return y


# -- recurrences with a decay per head or per channel -----------------------------------------------------------

def lightning_scan(proj: torch.Tensor, offsets, q_start, state_slots, state: torch.Tensor, decay: torch.Tensor,
                   heads: int, dim: int, vdim: int, chunked: int = 0, scan: bool = True) -> torch.Tensor:
    """o float32 [T, heads vdim] of the recurrence S <- decay_h S + k v^T, o = S^T q over a step's entries; q, k, v are
    the SiLU of ``proj``'s columns at ``offsets`` = (q, k, v); each request's S is its row of ``state`` float32
    [slots, heads * vdim * dim].  ``chunked`` > 0: entries of at least that many tokens run 64 tokens at a time on the
    matrix cores with q, k, v rounded to bfloat16 (key sizes 32, 64, 96, 128 and decays above zero only); ``scan``
    False then says that no entry is shorter, and the walk token by token is not launched."""
    _dev(proj, q_start, state_slots, state, decay)
    t = proj.shape[0]
    n_entries = state_slots.numel()
    off_q, off_k, off_v = (int(o) for o in offsets)
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1, "proj must be float32 [T, ld]")
    _need(min(off_q, off_k, off_v) >= 0 and max(off_q + heads * dim, off_k + heads * dim, off_v + heads * vdim)
          <= proj.shape[1], "the projections' columns do not fit proj")
    _need(dim <= 256, "lightning_scan: key sizes beyond 256 are not supported")
    _need(chunked == 0 or (chunked > 0 and dim % 32 == 0 and dim <= 128),
          "lightning_scan: the chunked kernel takes key sizes 32, 64, 96 and 128")
    _i32(q_start, "q_start", n_entries + 1)
    _i32(state_slots, "state_slots")
    _f32(decay, "decay", heads)
    _need(state.dtype is torch.float32 and state.is_contiguous() and state.dim() == 2
          and state.shape[1] == heads * vdim * dim, "the state must be float32 [slots, heads * vdim * dim]")
    o = torch.empty((t, heads * vdim), dtype=torch.float32, device=proj.device)
    _check(_module("lightning").atoma_lightning_scan(_p(proj), proj.stride(0) if t > 1 else proj.shape[1], off_q, off_k,
                                                     off_v, _p(q_start), _p(state_slots), _p(state), _p(decay), _p(o),
                                                     n_entries, heads, dim, vdim, int(chunked), int(bool(scan)),
                                                     _stream()), "lightning_scan")
    return o


def lightning_out(o: torch.Tensor, proj: torch.Tensor, off_g: int, w: torch.Tensor, eps: float,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """rmsnorm(o) * w * sigmoid(proj[:, off_g:]) in ``out_dtype``, the norm over all of a token's columns."""
    _dev(o, proj, w)
    t, n = o.shape
    _f32(o, "o")
    _f32(w, "norm weight", n)
    _need(proj.dtype is torch.float32 and proj.stride(1) == 1 and proj.shape[1] >= off_g + n, "the gates do not fit proj")
    y = torch.empty((t, n), dtype=out_dtype, device=o.device)
    _check(_module("lightning").atoma_lightning_out(_p(o), _p(proj), proj.stride(0) if t > 1 else proj.shape[1],
                                                    int(off_g), _p(w), ctypes.c_float(eps), _p(y), _code(y, "y"), t, n,
                                                    _stream()), "lightning_out")
    return y


def rglru_conv(proj: torch.Tensor, off_y: int, off_x: int, by, bx, conv, conv_b, token_seq, q_start, state_slots,
               state: torch.Tensor, width: int, taps: int):
    """(u, g) float32 [T, width]: the convolution of the x branch (its inputs before an entry from the request's row
    of ``state`` float32 [slots, taps * width], which also takes the inputs for the next step) and gelu of the y
    branch (see rglru.hip)."""
    _dev(proj, by, bx, conv, conv_b, token_seq, q_start, state_slots, state)
    t = proj.shape[0]
    n_entries = state_slots.numel()
    _need(proj.dtype is torch.float32 and proj.dim() == 2 and proj.stride(1) == 1
          and proj.shape[1] >= max(off_y, off_x) + width, "rglru: bad projection")
    for b, what in ((by, "y bias"), (bx, "x bias"), (conv_b, "convolution bias")):
        _f32(b, what, width)
    _f32(conv, "convolution", width * taps)
    _i32(token_seq, "token_seq", t)
    _i32(q_start, "q_start", n_entries + 1)
    _i32(state_slots, "state_slots")
    _need(state.dtype is torch.float32 and state.is_contiguous() and state.dim() == 2
          and state.shape[1] == taps * width, "the state must be float32 [slots, taps * width]")
    u = torch.empty((t, width), dtype=torch.float32, device=proj.device)
    g = torch.empty((t, width), dtype=torch.float32, device=proj.device)
    _check(_module("rglru").atoma_rglru_conv(_p(proj), proj.stride(0) if t > 1 else proj.shape[1], int(off_y), int(off_x),
                                             _p(by), _p(bx), _p(conv), _p(conv_b), _p(token_seq), _p(q_start),
                                             _p(state_slots), _p(state), _p(u), _p(g), t, n_entries, width, taps,
                                             _stream()), "rglru_conv")
    return u, g


def rglru_scan(gates: torch.Tensor, u: torch.Tensor, g: torch.Tensor, ba, bi, sp, q_start, state_slots,
               state: torch.Tensor, blocks: int, taps: int, out_dtype: torch.dtype, plan=None) -> torch.Tensor:
    """[T, width] = S * g with S <- a S + sqrt(1 - a^2) i u, a = exp(-8 r sp), r and i the sigmoids of ``gates``
    float32 [T, 2 width] (per block [r | i]) plus ``ba``, ``bi``.  ``plan``: (int32 device tensor, stretches) from
    ``mingru_plan`` for steps with long entries, or None for the plain walk."""
    _dev(gates, u, g, ba, bi, sp, q_start, state_slots, state)
    t, width = u.shape
    n_entries = state_slots.numel()
    _f32(gates, "gates", t * 2 * width)
    _f32(u, "u")
    _f32(g, "g", t * width)
    for b, what in ((ba, "gate bias"), (bi, "gate bias"), (sp, "softplus(lam)")):
        _f32(b, what, width)
    _i32(q_start, "q_start", n_entries + 1)
    _i32(state_slots, "state_slots")
    _need(state.dtype is torch.float32 and state.is_contiguous() and state.dim() == 2
          and state.shape[1] == taps * width and width % blocks == 0, "the state must be float32 [slots, taps * width]")
    out = torch.empty((t, width), dtype=out_dtype, device=u.device)
    arr, n_st, first, ab = None, 0, None, None
    if plan is not None and plan[1] > 0:
        arr, n_st = plan
        _i32(arr, "stretches", 3 * n_st + n_entries + 1)
        first = ctypes.c_void_p(arr.data_ptr() + 12 * n_st)
        ab = torch.empty((n_st, 2, width), dtype=torch.float32, device=u.device)
    _check(_module("rglru").atoma_rglru_scan(_p(gates), 2 * width, _p(u), _p(g), _p(ba), _p(bi), _p(sp), _p(q_start),
                                             _p(state_slots), _p(state), _p(arr), int(n_st),
                                             first if first is not None else _p(None), _p(ab), _p(out),
                                             _code(out, "out"), n_entries, width, int(blocks), int(taps), _stream()),
           "rglru_scan")
    return out


SPLIT_MAX_VOCAB = 262144       # the largest vocabulary whose rows ``sample_packed(split=True)`` cuts into parts


def sample_packed(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                  uniform: torch.Tensor, workspace: Optional[torch.Tensor] = None, split: bool = False,
                  cuts: bool = True) -> torch.Tensor:
    """Per row of float32 ``logits`` [S, V]: argmax where temperature <= 0, else a draw (see sampling.hip).

    Returns one float32 tensor [2, S]: row 0 holds the tokens (int32 bits), row 1 the logits of the chosen tokens,
    so that one copy brings both to the host.  ``split``: every row is shared by several blocks over six short
    launches instead of one long one (the same tokens; quicker when rows draw from a large vocabulary: one block
    walks a row with top-k and top-p in over 100 us); vocabularies beyond ``SPLIT_MAX_VOCAB`` keep the one launch.
    ``cuts=False`` (with ``split``): the caller knows that no row has a top-k or top-p cut, and the three launches
    that search for them are left out (``top_k`` and ``top_p`` are then not read).
    """
    _dev(logits, temperature, top_k, top_p, uniform)
    _need(logits.dim() == 2 and logits.dtype is torch.float32 and logits.stride(1) == 1, "logits must be float32 [S, V]")
    s, v = logits.shape
    for name, x, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                        ("top_p", top_p, torch.float32), ("uniform", uniform, torch.float32)):
        _need(x.dtype is dt and x.is_contiguous() and x.numel() == s, f"{name} must be {dt} [S]")
    if workspace is None:
        workspace = torch.empty((s, v), dtype=torch.float32, device=logits.device)
    _need(workspace.dtype is torch.float32 and workspace.is_contiguous() and workspace.numel() >= s * v,
          "sample: workspace too small")
    out = torch.empty((2, s), dtype=torch.float32, device=logits.device)
    ld = logits.stride(0) if s > 1 else v
    if split and v <= SPLIT_MAX_VOCAB:
        lib = core()
        lib.atoma_sample_split_scratch_bytes.restype = ctypes.c_size_t
        scratch = torch.empty((int(lib.atoma_sample_split_scratch_bytes(s)) + 3) // 4, dtype=torch.int32,
                              device=logits.device)
        _check(lib.atoma_sample_split(_p(logits), ld, s, v, _p(temperature), _p(top_k), _p(top_p), _p(uniform),
                                      _p(workspace), _p(scratch), 1 if cuts else 0, _p(out[0]), _p(out[1]), _stream()),
               "sample (split)")
        return out
    _check(core().atoma_sample(_p(logits), ld, s, v, _p(temperature), _p(top_k),
                               _p(top_p), _p(uniform), _p(workspace), _p(out[0]), _p(out[1]), _stream()), "sample")
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, workspace: Optional[torch.Tensor] = None, split: bool = False, cuts: bool = True):
    """``sample_packed`` as (tokens int32 [S], logits of the chosen tokens float32 [S])."""
    out = sample_packed(logits, temperature, top_k, top_p, uniform, workspace, split, cuts)
    return out[0].view(torch.int32), out[1]


def repeat_penalty(logits: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor, penalty: torch.Tensor) -> None:
    """In place: for each pair (rows[i], tokens[i]) the logit is divided (if >= 0) or multiplied by penalty[row]."""
    _dev(logits, rows, tokens, penalty)
    _need(logits.dim() == 2 and logits.dtype is torch.float32 and logits.stride(1) == 1, "logits must be float32 [S, V]")
    n = rows.numel()
    _i32(rows, "rows")
    _i32(tokens, "tokens", n)
    _need(penalty.dtype is torch.float32 and penalty.numel() == logits.shape[0], "penalty must be float32 [S]")
    _check(core().atoma_repeat_penalty(_p(logits), logits.stride(0), _p(rows), _p(tokens), _p(penalty), n, _stream()),
           "repeat_penalty")


def feed_tokens(dst: torch.Tensor, src: torch.Tensor, pairs: torch.Tensor) -> None:
    """dst[pairs[i, 0]] = src[pairs[i, 1]] for int32 device tensors; the caller guarantees the indices' ranges."""
    _dev(dst, src, pairs)
    _i32(dst, "dst")
    _i32(src, "src")
    _need(pairs.dtype is torch.int32 and pairs.is_contiguous() and pairs.dim() == 2 and pairs.shape[1] == 2,
          "pairs must be contiguous int32 [n, 2]")
    _check(core().atoma_feed_tokens(_p(dst), _p(src), _p(pairs), pairs.shape[0], _stream()), "feed_tokens")


def measure_device_peaks(device: Optional[torch.device] = None, size_bytes: int = 1 << 30) -> dict:
    """What the GPU delivers, measured with the probes of ``microbench.hip``: GB/s of a read stream and of a copy
    (bytes read plus bytes written) over device memory, and TFLOP/s of a loop of bfloat16 MFMAs.

    The read stream is the yardstick that no kernel of this repository may beat, so it is the best of a sweep: 4, 8
    and 16 loads of 16 bytes in flight a thread, 4 to 32 workgroups a CU, over ``size_bytes`` and over four times as
    much (``hbm_read_how`` says which won)."""
    lib = load_hip_module("microbench")
    dev = device or torch.device("cuda:0")
    big = 4 * size_bytes
    src = torch.empty(big, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty(size_bytes, dtype=torch.uint8, device=dev)
    sink = torch.zeros(4, dtype=torch.float32, device=dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count

    def best(launch, reps=5):
        launch()
        torch.cuda.synchronize(dev)
        times = []
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            launch()
            b.record()
            torch.cuda.synchronize(dev)
            times.append(a.elapsed_time(b) * 1e-3)
        return min(times)

    out = {}
    with torch.cuda.device(dev):
        reads = []
        for nbytes in (size_bytes, big):
            for per_cu in (4, 8, 16, 32):
                for u in (4, 8, 16):
                    t = best(lambda: _check(lib.atoma_probe_read(_p(src), ctypes.c_size_t(nbytes), cus * per_cu, u,
                                                                 _p(sink), _stream()), "probe_read"), reps=3)
                    reads.append((nbytes / t / 1e9, f"{nbytes >> 20} MiB, {per_cu} workgroups a CU, {u} loads in flight"))
        copy = min(best(lambda g=g: _check(lib.atoma_probe_copy(_p(src), _p(dst), ctypes.c_size_t(size_bytes), g,
                                                                 _stream()), "probe_copy")) for g in (cus * 8, cus * 16))
        iters, grid = 20000, cus * 8
        mfma = best(lambda: _check(lib.atoma_probe_mfma(iters, grid, _p(sink), _stream()), "probe_mfma"), reps=3)
    rate, how = max(reads)
    out["hbm_read_gbs"] = round(rate, 1)
    out["hbm_read_how"] = how
    out["hbm_copy_gbs"] = round(2 * size_bytes / copy / 1e9, 1)
    out["mfma_bf16_tflops"] = round(grid * 4 * iters * 4 * 2 * 32 * 32 * 16 / mfma / 1e12, 1)
    return out


def measure_chain_floors(device: Optional[torch.device] = None) -> dict:
    """What a chain of dependent kernels costs on this GPU beyond its bytes, in microseconds a kernel (the probes of
    ``microbench.hip``, each launched 32 times in a row inside one graph, every launch over other memory, so that
    nothing comes from a cache): an empty kernel behind another; a read stream of 8, 16, 32 and 64 MB (the sizes of a
    decode step's weight matrices); and a barrier over a grid of one workgroup a CU inside one kernel, which is what
    a persistent kernel would pay where the chain pays a launch."""
    lib = load_hip_module("microbench")
    dev = device or torch.device("cuda:0")
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    n = 32
    out = {}
    with torch.cuda.device(dev):
        src = torch.empty(n * (64 << 20), dtype=torch.uint8, device=dev).random_(0, 255)
        sink = torch.zeros(4, dtype=torch.float32, device=dev)
        base = src.data_ptr()

        def chain(nbytes: int) -> float:
            def launches():
                for i in range(n):
                    _check(lib.atoma_probe_read(ctypes.c_void_p(base + i * (64 << 20)), ctypes.c_size_t(nbytes), cus * 2,
                                                4, _p(sink), _stream()), "probe_read")
            launches()
            torch.cuda.synchronize(dev)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                launches()
            graph.replay()
            torch.cuda.synchronize(dev)
            best = float("inf")
            for _ in range(4):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                graph.replay()
                b.record()
                torch.cuda.synchronize(dev)
                best = min(best, a.elapsed_time(b) * 1e3 / n)
            return round(best, 2)

        out["empty_kernel_us"] = chain(0)
        for mb in (8, 16, 32, 64):
            out[f"read_{mb}mb_us"] = chain(mb << 20)
        nb = 2000
        best = float("inf")
        for _ in range(3):
            ctrl = torch.zeros(128, dtype=torch.int32, device=dev)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            _check(lib.atoma_probe_barrier(_p(ctrl), cus, nb, _stream()), "probe_barrier")
            b.record()
            torch.cuda.synchronize(dev)
            if int(ctrl[64]) != 0:
                raise KernelError("probe_barrier: a wait ran out (the grid was not resident at once)")
            best = min(best, a.elapsed_time(b) * 1e3 / nb)
        out["grid_barrier_us"] = round(best, 2)
    return out
