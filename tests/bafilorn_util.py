"""Shared pieces of the Bafilorn tests: small configurations that differ from each other in every size, and the plain
model's weights as numpy arrays."""
from __future__ import annotations

import math
import os

import numpy as np
import torch


def latent(dim=16, heads=4, kv_rank=40, q_rank=24, rot_dim=8, vdim=24, scale=0.2, base=100.0, rot_dims=None):
    m = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot_dim": rot_dim, "vdim": vdim,
         "scale": scale}
    if rot_dim:
        m["rot"] = {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}
    return m


def lightning(heads=3, dim=16, vdim=24, decay=None):
    return {"decay": list(decay) if decay is not None else [0.5 + 0.49 * (h + 1) / heads for h in range(heads)],
            "dim": dim, "heads": heads, "vdim": vdim}


def parallel(dim=32, heads=4, kv_heads=2, scale=0.2, mask=7, rot_dims=16, base=100.0, scaling=None, width=48, blocks=3,
             conv=3):
    left = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": dim, "scale": scale}
    if mask:
        left["mask"] = {"size": mask}
    if rot_dims:
        left["rot"] = {"base": base, "dims": rot_dims}
        if scaling is not None:
            left["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"left": left, "right": {"blocks": blocks, "conv": conv, "width": width}}


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=64, vocab=97, eps=1e-5, streams=2, bigram=(53, 7, 3), scale=3.0, loop=None):
    c = {"architecture": "Bafilorn", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width,
         "embedding": {"scale": scale}}
    if bigram is not None:
        c["embedding"]["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}
    if streams is not None:
        c["streams"] = streams
    if loop is not None:
        c["loop"] = dict(zip(("start", "stop", "times"), loop))
    return c


# two copies of the stream; a recurrence first; chunks of 7; slowed long waves; a layer without a feed-forward; the last
# two layers run twice
BAF_A = config([
    layer("lightning", lightning(heads=3, dim=16, vdim=24), 48),
    layer("parallel", parallel(dim=32, heads=4, kv_heads=2, scale=0.2, mask=7, rot_dims=16, base=100.0,
                               scaling=(4.0, 64, 8.0, 1.0), width=48, blocks=3, conv=3), None),
    layer("latent_attention", latent(dim=16, heads=4, kv_rank=40, q_rank=24, rot_dim=8, vdim=24, scale=0.2), 40),
], width=64, vocab=97, streams=2, loop=(1, 3, 2))
# four copies; no table of pairs and no scale; heads of 64 columns (the matrix-core attention as it is) with every
# column rotated and no slowing; only half of the latent's rotated part turns; one block and one tap in the
# recurrence; one head of lightning attention; no loop
BAF_B = config([
    layer("latent_attention", latent(dim=32, heads=2, kv_rank=64, q_rank=48, rot_dim=32, rot_dims=16, vdim=16, scale=0.15,
                                     base=500.0), 96),
    layer("parallel", parallel(dim=64, heads=8, kv_heads=4, scale=0.125, mask=33, rot_dims=64, base=500.0, width=256,
                               blocks=1, conv=1), 64),
    layer("lightning", lightning(heads=1, dim=128, vdim=64, decay=[0.97]), 32),
], width=128, vocab=211, eps=3e-6, streams=4, bigram=None, scale=1.0)
# no copies at all (the plain residual); sizes that are no multiple of anything; all key heads their own; a rotated
# part of the latent that is not rotated; the first layer runs three times
BAF_C = config([
    layer("parallel", parallel(dim=20, heads=3, kv_heads=3, scale=0.3, mask=11, rot_dims=10, base=30.0,
                               scaling=(2.0, 16, 4.0, 2.0), width=30, blocks=5, conv=4), 24),
    layer("latent_attention", latent(dim=10, heads=3, kv_rank=20, q_rank=12, rot_dim=6, rot_dims=0, vdim=6, scale=0.4), None),
    layer("lightning", lightning(heads=2, dim=10, vdim=5, decay=[1.0, 0.3]), 20),
], width=40, vocab=50, streams=None, bigram=(11, 1, 1), scale=0.5, loop=(0, 1, 3))
# one of everything: one copy (with its tensors), one head, one block, no chunks, no rotation on the left
BAF_D = config([
    layer("latent_attention", latent(dim=8, heads=1, kv_rank=16, q_rank=8, rot_dim=2, vdim=8, scale=1.0, base=2.0), 16),
    layer("parallel", parallel(dim=16, heads=1, kv_heads=1, scale=0.25, mask=None, rot_dims=0, width=8, blocks=1,
                               conv=2), 16),
    layer("lightning", lightning(heads=1, dim=1, vdim=1, decay=[0.9]), None),
], width=32, vocab=30, streams=1, bigram=(1, 5, 9), scale=2.0)


def random_config(rng):
    """A configuration drawn from ``rng`` (a ``random.Random``): two to eight layers of the three kinds in any order,
    sizes that are and are not multiples of what the kernels like, every optional key present or absent."""
    return rand_cfg(rng)


def rand_cfg(rng):
    width = rng.choice([96, 128, 192, 256, 320, 384])
    kinds = ["latent_attention", "lightning", "parallel"]
    n = rng.randint(2, 5)
    order = [rng.choice(kinds) for _ in range(n)]
    for k in kinds:
        if k not in order and rng.random() < 0.7: order.append(k)
    layers = []
    for k in order:
        ff = rng.choice([0, 64, 100, 256, 384]) if rng.random() < 0.85 else 0
        if k == "latent_attention":
            rd = rng.choice([0, 2, 8, 16, 32, 64])
            rank = rng.choice([16, 24, 48, 96, 128, 160])
            if rank + rd > 256: rank = 256 - rd
            dims = rd if rng.random() < 0.7 else rng.choice([d for d in (0, 2, 4, 8, 16, 32) if d <= rd])
            m = latent(dim=rng.choice([8, 16, 24, 32, 64]), heads=rng.choice([1, 2, 3, 4, 8, 12]), kv_rank=rank,
                       q_rank=rng.choice([8, 32, 64, 128, 200]), rot_dim=rd, vdim=rng.choice([8, 16, 32, 48, 64]),
                       scale=rng.choice([0.1, 0.15, 0.2]), base=rng.choice([100.0, 10000.0, 50000.0]), rot_dims=dims)
        elif k == "lightning":
            h = rng.choice([1, 2, 4, 6, 8])
            m = lightning(heads=h, dim=rng.choice([8, 16, 32, 48, 64, 96, 128, 160]), vdim=rng.choice([8, 16, 24, 32, 64, 100]),
                          decay=[math.exp(-1.0 / (2.0 ** (i + rng.random()))) if rng.random() < 0.9 else 0.999 for i in range(h)])
        else:
            kvh = rng.choice([1, 2, 4])
            g = rng.choice([1, 2, 4, 8])
            dim = rng.choice([16, 32, 40, 64, 80, 128])
            rot = rng.choice([0, 8, 16, dim])
            if rot > dim: rot = dim
            sc = None if rng.random() < 0.3 else (rng.choice([2.0, 4.0, 8.0, 16.0]), rng.choice([64, 512, 2048, 4096]), rng.choice([8.0, 32.0, 64.0]), rng.choice([0.5, 1.0, 2.0]))
            bw = rng.choice([64, 128, 256, 96])
            blocks = rng.choice([b for b in (1, 2, 4, 8, 3) if bw % b == 0])
            m = parallel(dim=dim, heads=kvh * g, kv_heads=kvh, scale=rng.choice([0.125, 0.1, 0.2]), mask=rng.choice([None, 5, 16, 37, 64, 100, 150]),
                         rot_dims=rot, base=rng.choice([1000.0, 30000.0, 500000.0]), scaling=sc if rot else None, width=bw, blocks=blocks,
                         conv=rng.choice([1, 2, 3, 4, 5, 7]))
        layers.append(layer(k, m, ff))
    loop = None
    if rng.random() < 0.7:
        a = rng.randint(0, len(layers) - 1); b = rng.randint(a + 1, len(layers))
        loop = (a, b, rng.choice([1, 2, 3]))
    bg = None if rng.random() < 0.2 else (rng.choice([7, 101, 521, 4099]), rng.choice([1, 29, 1009, 65537]), rng.choice([1, 19, 257, 40503]))
    return config(layers, width=width, vocab=rng.choice([50, 97, 300, 450, 1000]), eps=rng.choice([1e-6, 1e-5]),
                  streams=rng.choice([None, 1, 2, 3, 4, 5]), bigram=bg, scale=rng.choice([1.0, 10.0, 0.5]), loop=loop)


def numpy_weights(path: str):
    from safetensors.torch import load_file
    return {k: v.to(torch.float64).numpy() for k, v in load_file(os.path.join(path, "model.safetensors")).items()}


def as_numpy(w: dict, prefix: str = ""):
    """A dict of torch tensors as float64 numpy arrays, the names behind ``prefix``."""
    return {prefix + k: np.asarray(v.to(torch.float64)) for k, v in w.items()}
