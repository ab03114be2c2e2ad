"""A plain, slow Bafilorn: one function per mechanism, numpy float64, whole sequences at once or token by token.

It shares no code with the engine.  ``cfg`` is the JSON object of a config.json, ``w`` a dict of float64 arrays by
checkpoint name.  Notation: h [T, width] is a sublayer's input, p the positions 0 .. T-1 of one sequence.
"""
from __future__ import annotations

import math

import numpy as np


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


# ---------------------------------------------------------------------------------------------------- embedding

def embed(tokens, w, cfg):
    """scale * embed[token] + bigram[row]; row = (prev * mul_prev + token * mul_cur) mod buckets, the table's last row
    for a sequence's first token."""
    e = cfg["embedding"]
    x = w["embed"][tokens] * e["scale"]
    bg = e.get("bigram")
    if bg is not None:
        rows = np.empty(len(tokens), dtype=np.int64)
        for t, tok in enumerate(tokens):
            rows[t] = bg["buckets"] if t == 0 else (int(tokens[t - 1]) * bg["mul_prev"] + int(tok) * bg["mul_cur"]) \
                % bg["buckets"]
        x = x + w["bigram"][rows]
    return x


# ---------------------------------------------------------------------------------------------------- rotations

def plain_frequencies(base, dims):
    return np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])


def yarn_frequencies(base, dims, sc):
    """(frequencies, factor on cos and sin) with the band-wise slow-down of rot.scaling."""
    f = plain_frequencies(base, dims)
    if sc is None:
        return f, 1.0

    def where(turns):
        return dims * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(where(sc["fast"])), 0)
    hi = min(math.ceil(where(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x, p, freqs, dims, layout, mag=1.0):
    """x [T, heads, d]: the first ``dims`` columns of every head turned by p * freqs; 'interleaved' pairs (2i, 2i + 1),
    'half' pairs (i, i + dims / 2)."""
    out = x.copy()
    ang = np.asarray(p, dtype=np.float64)[:, None] * freqs[None, :]            # [T, dims / 2]
    c, s = (np.cos(ang) * mag)[:, None, :], (np.sin(ang) * mag)[:, None, :]
    if layout == "interleaved":
        ia, ib = np.arange(0, dims, 2), np.arange(1, dims, 2)
    else:
        ia, ib = np.arange(dims // 2), np.arange(dims // 2) + dims // 2
    u, v = x[..., ia], x[..., ib]
    out[..., ia] = u * c - v * s
    out[..., ib] = v * c + u * s
    return out


# ---------------------------------------------------------------------------------------------------- attention

def softmax_attention(q, k, v, p, scale, chunk=None, sink=False):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads key head h // (H / G).  Position i sees j <= i, with
    ``chunk`` only those of its own chunk; ``sink`` adds one to the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        pi, pj = np.asarray(p)[:, None], np.asarray(p)[None, :]
        vis = pj <= pi
        if chunk:
            vis &= (pi // chunk) == (pj // chunk)
        s = np.where(vis, s, -np.inf)
        m = np.maximum(s.max(axis=1, keepdims=True), 0.0 if sink else -np.inf)
        e = np.exp(s - m)
        den = e.sum(axis=1, keepdims=True) + (np.exp(-m) if sink else 0.0)
        out[:, h] = (e / den) @ v[:, g]
    return out


def latent_attention(h, p, w, pre, m, eps):
    H, d, r, dv, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    cq = unit_rms(h @ w[pre + "dq"].T, eps) * w[pre + "dq.norm"]
    q = (cq @ w[pre + "uq"].T).reshape(T, H, d + r)
    dkv = h @ w[pre + "dkv"].T
    c = unit_rms(dkv[:, :kr], eps) * w[pre + "dkv.norm"]
    k_rot = dkv[:, kr:].reshape(T, 1, r)
    q_rot = q[..., d:]
    rot = m.get("rot")
    if rot is not None and rot["dims"]:
        f = plain_frequencies(rot["base"], rot["dims"])
        q_rot = rotate(q_rot, p, f, rot["dims"], "interleaved")
        k_rot = rotate(k_rot, p, f, rot["dims"], "interleaved")
    k = np.concatenate([(c @ w[pre + "uk"].T).reshape(T, H, d), np.repeat(k_rot, H, axis=1)], axis=2)
    v = (c @ w[pre + "uv"].T).reshape(T, H, dv)
    qq = np.concatenate([q[..., :d], q_rot], axis=2)
    o = softmax_attention(qq, k, v, p, m["scale"]).reshape(T, H * dv)
    o = o * sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def tied_value_attention(h, p, w, pre, m):
    """The left branch: grouped heads, values are the keys as projected, biases, half-split rotation with band-wise
    scaling, chunks, a sink of score zero, an output gate."""
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    T = h.shape[0]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, d)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, d)
    v = k.copy()
    rot = m.get("rot")
    if rot is not None and rot["dims"]:
        f, mag = yarn_frequencies(rot["base"], rot["dims"], rot.get("scaling"))
        q = rotate(q, p, f, rot["dims"], "half", mag)
        k = rotate(k, p, f, rot["dims"], "half", mag)
    chunk = m["mask"]["size"] if m.get("mask") else None
    o = softmax_attention(q, k, v, p, m["scale"], chunk=chunk, sink=True).reshape(T, H * d)
    o = o * sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T + w[pre + "o.b"]


# ---------------------------------------------------------------------------------------------------- recurrences

def lightning(h, w, pre, m, eps, state=None):
    """Per head S <- decay S + k v^T, o = S^T q, with q, k, v through SiLU.  Returns (output, state [H, d, dv])."""
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ w[pre + "q"].T).reshape(T, H, d)
    k = silu(h @ w[pre + "k"].T).reshape(T, H, d)
    v = silu(h @ w[pre + "v"].T).reshape(T, H, dv)
    S = np.zeros((H, d, dv)) if state is None else state.copy()
    o = np.zeros((T, H, dv))
    decay = np.asarray(m["decay"], dtype=np.float64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(o.reshape(T, H * dv), eps) * w[pre + "norm"]
    o = o * sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T, S


def gated_linear_recurrence(h, w, pre, m, state=None):
    """The right branch.  ``state`` = (the last taps - 1 inputs of the convolution [taps - 1, width], S [width])."""
    width, taps, blocks = m["width"], m["conv"], m["blocks"]
    T = h.shape[0]
    y = gelu_tanh(h @ w[pre + "y"].T + w[pre + "y.b"])
    xin = h @ w[pre + "x"].T + w[pre + "x.b"]
    tail, S = (np.zeros((taps - 1, width)), np.zeros(width)) if state is None else (state[0].copy(), state[1].copy())
    padded = np.concatenate([tail, xin], axis=0)
    cw = w[pre + "conv"]                                             # [channels, taps], last column: current token
    u = np.zeros((T, width))
    for t in range(T):
        u[t] = (padded[t: t + taps].T * cw).sum(axis=1) + w[pre + "conv.b"]
    bs = width // blocks
    out = np.zeros((T, width))
    sp = softplus(w[pre + "lam"])
    for t in range(T):
        r, i = np.zeros(width), np.zeros(width)
        for b in range(blocks):
            ub = u[t, b * bs: (b + 1) * bs]
            r[b * bs: (b + 1) * bs] = sigmoid(w[pre + "ra"][b] @ ub + w[pre + "ra.b"][b])
            i[b * bs: (b + 1) * bs] = sigmoid(w[pre + "ri"][b] @ ub + w[pre + "ri.b"][b])
        a = np.exp(-8.0 * r * sp)
        S = a * S + np.sqrt(1.0 - a * a) * i * u[t]
        out[t] = S * y[t]
    new_tail = padded[padded.shape[0] - (taps - 1):] if taps > 1 else tail
    return out @ w[pre + "o"].T, (new_tail, S)


def parallel(h, p, w, pre, m, eps, state=None):
    left = tied_value_attention(h, p, w, pre + "left.", m["left"])
    right, st = gated_linear_recurrence(h, w, pre + "right.", m["right"], state)
    return 0.5 * (unit_rms(left, eps) * w[pre + "left.out"] + unit_rms(right, eps) * w[pre + "right.out"]), st


# ---------------------------------------------------------------------------------------------------- the rest

def feed_forward(h, w, pre):
    return np.maximum(h @ w[pre + "up"].T, 0.0) ** 2 @ w[pre + "down"].T


def norm_one_plus(x, wt, eps):
    return unit_rms(x, eps) * (1.0 + wt)


def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    lo, hi = loop["start"], loop["stop"]
    return list(range(lo)) + list(range(lo, hi)) * loop["times"] + list(range(hi, n))


def mixer(kind, h, p, w, pre, m, eps):
    if kind == "latent_attention":
        return latent_attention(h, p, w, pre, m, eps)
    if kind == "lightning":
        return lightning(h, w, pre, m, eps)[0]
    if kind == "parallel":
        return parallel(h, p, w, pre, m, eps)[0]
    raise ValueError(kind)


def forward(tokens, w, cfg):
    """(logits [T, vocab], the stream after every layer run [runs, T, width]) for one whole sequence."""
    eps = cfg["norm"]["eps"]
    p = np.arange(len(tokens))
    x0 = embed(np.asarray(tokens), w, cfg)
    copies = cfg.get("streams")                 # absent: one stream and no connection tensors
    s = int(copies or 1)
    xs = [x0.copy() for _ in range(s)]
    seen = []
    for li in run_order(cfg):
        layer = cfg["layers"][li]
        pre = f"l{li}."
        subs = [(1, lambda h: mixer(layer["type"], h, p, w, pre + "mix.", layer["mixer"], eps))]
        if layer.get("mlp") is not None:
            subs.append((2, lambda h: feed_forward(h, w, pre + "mlp.")))
        for q, fn in subs:
            if copies is not None:
                hin, hmix, hout = w[pre + f"hc{q}.in"], w[pre + f"hc{q}.mix"], w[pre + f"hc{q}.out"]
                u = sum(hin[i] * xs[i] for i in range(s))
                y = fn(norm_one_plus(u, w[pre + f"norm{q}"], eps))
                xs = [sum(hmix[i, t] * xs[i] for i in range(s)) + hout[t] * y for t in range(s)]
            else:
                xs = [xs[0] + fn(norm_one_plus(xs[0], w[pre + f"norm{q}"], eps))]
        seen.append(sum(xs))
    x = norm_one_plus(sum(xs), w["final.norm"], eps)
    return x @ w["head"].T, np.stack(seen)
