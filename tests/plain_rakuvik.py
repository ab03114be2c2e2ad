"""A plain, slow Rakuvik decoder on the CPU: the yardstick of the engine's tests for that design.

Whole sequences, token by token where the design is recurrent, no cache, no batching, one function per mechanism.
Nothing here is imported from the framework.  Weights are a ``dict`` from the checkpoint's tensor names to CPU
tensors of the working dtype (float64 by default); the configuration is the plain ``dict`` of config.json.

The design in this file's notation (x: a token's residual row, h: a sublayer's input, N_g(v) = v / sqrt(mean(v^2) +
eps) * g with ONE number g per norm):

* layer i:    y = x + N_1b(mixer(N_1(x)));  X_(i+1) = y + N_2b(ff(N_2(y)))  (no second half without a feed-forward);
              the next layer (or the output) reads  x = sum_(j <= i+1) dwa_i[j] X_j,  X_0 the embedding's rows
* attention:  every head has two score maps (q1, k1), (q2, k2) over one set of values; the first ``rot.dims``
              columns of each map are turned in pairs (c, c + dims/2) by p * base^(-2c/dims) / factor; each map is a
              causal softmax attention a1, a2; o = a1 - lam a2, lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff;
              o / sqrt(mean(o^2) + eps) * (1 - diff), times sigmoid(W_g h)_head, then W_o.  ``kv_from: j`` reads the
              rotated keys and the values that layer j made
* mingru:     z = sigmoid(W_z h + b_z), u = W_x h + b_x, c = u + 1/2 (u >= 0) or sigmoid(u) (u < 0);
              S <- (1 - z) S + z c from S = 0;  out = W_o (S * silu(W_g h))
* dense ff:   W_down (gelu_tanh(W_gate h) * (W_up h))
* moe ff:     s = softmax(W_r h); the ``top`` largest of s + correction are chosen and weighed by s * scale (not
              renormalised); experts W_down relu(W_up h)^2; a shared expert of the same form, times sigmoid(W_sg h)
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

W = Dict[str, torch.Tensor]


def scalar_norm(x: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * g


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def linear_scaled_frequencies(base: float, dims: int, factor: float, dtype=torch.float64) -> torch.Tensor:
    c = torch.arange(dims // 2, dtype=dtype)
    return torch.tensor(float(base), dtype=dtype) ** (-2.0 * c / dims) / factor


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """x [T, maps, dim]: column c < dims/2 is paired with column c + dims/2 (dims = 2 len(freq)) and the pair is
    turned by positions * freq_c; the columns from dims on pass."""
    half = freq.numel()
    if half == 0:
        return x.clone()
    ang = positions.to(x.dtype)[:, None] * freq.to(x.dtype)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    u, v = x[..., :half], x[..., half:2 * half]
    out[..., :half] = u * c - v * s
    out[..., half:2 * half] = v * c + u * s
    return out


def frequencies_of(m: dict, dtype=torch.float64) -> torch.Tensor:
    rot = m.get("rot")
    if not rot or not rot.get("dims"):
        return torch.zeros(0, dtype=dtype)
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    return linear_scaled_frequencies(rot["base"], rot["dims"], factor, dtype)


def keys_and_values(h: torch.Tensor, w: W, pre: str, m: dict):
    """(k [T, kv_heads, 2, dim] rotated, v [T, kv_heads, vdim]) of a layer that owns its projections."""
    t = h.shape[0]
    g, dim, vdim = m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(t)
    k = (h @ w[pre + "k"].T).view(t, g * 2, dim)
    k = rotate_halves(k, pos, frequencies_of(m, h.dtype)).view(t, g, 2, dim)
    v = (h @ w[pre + "v"].T).view(t, g, vdim)
    return k, v


def difference_weight(w: W, pre: str, m: dict) -> float:
    return float(torch.exp((w[pre + "lq1"] * w[pre + "lk1"]).sum()) - torch.exp((w[pre + "lq2"] * w[pre + "lk2"]).sum())
                 + m["diff"])


def differential_attention(h: torch.Tensor, w: W, pre: str, m: dict, eps: float, kv=None) -> torch.Tensor:
    """The 'attention' mixer on a whole sequence h [T, width] (positions 0 .. T-1).  ``kv``: another layer's
    (k, v) where this one has none of its own."""
    t = h.shape[0]
    nh, g, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(t)
    q = rotate_halves((h @ w[pre + "q"].T).view(t, nh * 2, dim), pos, frequencies_of(m, h.dtype)).view(t, nh, 2, dim)
    k, v = keys_and_values(h, w, pre, m) if kv is None else kv
    lam = difference_weight(w, pre, m)
    gate = torch.sigmoid(h @ w[pre + "g"].T)                         # [T, heads]
    seen = torch.tril(torch.ones(t, t, dtype=torch.bool))
    heads = []
    for a in range(nh):
        b = a // (nh // g)
        maps = []
        for j in range(2):
            s = (q[:, a, j] @ k[:, b, j].T) * m["scale"]
            s = s.masked_fill(~seen, float("-inf"))
            maps.append(torch.softmax(s, dim=-1) @ v[:, b])
        o = maps[0] - lam * maps[1]
        o = o / torch.sqrt((o * o).mean(dim=-1, keepdim=True) + eps) * (1.0 - m["diff"])
        heads.append(o * gate[:, a:a + 1])
    return torch.cat(heads, dim=-1) @ w[pre + "o"].T


def mingru(h: torch.Tensor, w: W, pre: str, m: dict) -> torch.Tensor:
    """The 'mingru' mixer, token by token from a zero state."""
    z = torch.sigmoid(h @ w[pre + "z"].T + w[pre + "z.b"])
    u = h @ w[pre + "x"].T + w[pre + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    s = torch.zeros(m["width"], dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        s = (1.0 - z[t]) * s + z[t] * cand[t]
        rows.append(s)
    return (torch.stack(rows) * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def dense_ff(h: torch.Tensor, w: W, pre: str) -> torch.Tensor:
    return (gelu_tanh(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def squared_relu_expert(h: torch.Tensor, w: W, pre: str) -> torch.Tensor:
    return torch.relu(h @ w[pre + "up"].T) ** 2 @ w[pre + "down"].T


def route(h: torch.Tensor, w: W, pre: str, r: dict):
    """(ids [T, top], weights [T, top]): chosen by score plus correction, weighed by the score alone."""
    s = torch.softmax(h @ w[pre + "router"].T, dim=-1)
    ids = torch.topk(s + w[pre + "correction"], r["top"], dim=-1).indices
    return ids, torch.gather(s, 1, ids) * r["scale"]


def moe_ff(h: torch.Tensor, w: W, pre: str, mlp: dict) -> torch.Tensor:
    ids, weights = route(h, w, pre, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, p in zip(ids[t].tolist(), weights[t]):
            out[t] += p * squared_relu_expert(h[t:t + 1], w, f"{pre}e{e}.")[0]
    if mlp.get("shared"):
        out = out + squared_relu_expert(h, w, pre + "shared.") * torch.sigmoid(h @ w[pre + "shared.sg"].T)
    return out


def feed_forward(h: torch.Tensor, w: W, pre: str, mlp: dict) -> torch.Tensor:
    return dense_ff(h, w, pre) if mlp["kind"] == "dense" else moe_ff(h, w, pre, mlp)


def forward(tokens: List[int], w: W, cfg: dict, dtype=torch.float64, streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence.  ``streams`` (a list) receives every layer's result X_(i+1)."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    results = [x]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = scalar_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = keys_and_values(h, w, p + "mix.", m)
                a = differential_attention(h, w, p + "mix.", m, eps)
            else:
                a = differential_attention(h, w, p + "mix.", m, eps, kv=kept[m["kv_from"]])
        elif layer["type"] == "mingru":
            a = mingru(h, w, p + "mix.", m)
        else:
            raise ValueError(f"unknown layer type {layer['type']}")
        x = x + scalar_norm(a, w[p + "norm1b"], eps)
        if layer.get("mlp"):
            f = feed_forward(scalar_norm(x, w[p + "norm2"], eps), w, p + "mlp.", layer["mlp"])
            x = x + scalar_norm(f, w[p + "norm2b"], eps)
        results.append(x)
        if streams is not None:
            streams.append(x)
        x = sum(w[p + "dwa"][j] * results[j] for j in range(i + 2))
    return scalar_norm(x, w["final.norm"], eps) @ w["head"].T


def greedy_generate(prompt: List[int], n: int, w: W, cfg: dict) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(toks, w, cfg)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out
