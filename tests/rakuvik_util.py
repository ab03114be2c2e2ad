"""Shared pieces of the Rakuvik tests: small configurations that differ from each other in every size."""
from __future__ import annotations


def attention(dim=16, heads=4, kv_heads=2, vdim=32, scale=0.25, diff=0.25, rot_dims=8, base=1000.0, factor=None,
              kv_from=None):
    m = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim, "scale": scale, "diff": diff}
    if rot_dims is not None:
        m["rot"] = {"base": base, "dims": rot_dims}
        if factor is not None:
            m["rot"]["scaling"] = {"factor": factor}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def mingru(width=48):
    return {"width": width}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def moe(ff=32, experts=4, top=2, scale=1.5, shared=32):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "scale": scale, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=64, vocab=97, eps=1e-5):
    return {"architecture": "Rakuvik", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


# the recurrence first; two maps of 16 columns under values of 24 (no multiple of 16), half of a map rotated and
# slowed fourfold; a layer that reads the cache of the layer before it; one layer without a feed-forward; three
# experts of which one is chosen, without a shared expert
RAK_A = config([
    layer("mingru", mingru(40), moe(ff=32, experts=3, top=1, scale=0.7, shared=0)),
    layer("attention", attention(dim=16, heads=4, kv_heads=2, vdim=24, scale=0.3, diff=0.2, rot_dims=8, base=100.0,
                                 factor=4.0), dense(40)),
    layer("attention", attention(dim=16, heads=4, kv_heads=2, vdim=24, scale=0.3, diff=0.2, rot_dims=8, base=100.0,
                                 factor=4.0, kv_from=1), None),
    layer("mingru", mingru(72), moe(ff=64, experts=6, top=2, scale=2.0, shared=32)),
], width=64, vocab=97)
# heads of 2 x 32 columns over values of 64 (the matrix-core attention in bfloat16 as it is), every head its own keys,
# the whole map rotated without slowing; a recurrence wider than the stream; all experts chosen; an attention layer that
# rotates nothing; two layers that read the first layer's cache
RAK_B = config([
    layer("attention", attention(dim=32, heads=4, kv_heads=4, vdim=64, scale=0.18, diff=0.4, rot_dims=32, base=500.0),
          moe(ff=32, experts=4, top=4, scale=0.5, shared=64)),
    layer("mingru", mingru(192), dense(96)),
    layer("attention", attention(dim=32, heads=4, kv_heads=4, vdim=64, scale=0.18, diff=0.4, rot_dims=32, base=500.0,
                                 kv_from=0), dense(64)),
    layer("attention", attention(dim=64, heads=2, kv_heads=1, vdim=32, scale=0.12, diff=0.1, rot_dims=None),
          moe(ff=96, experts=8, top=3, scale=1.0, shared=32)),
    layer("attention", attention(dim=32, heads=4, kv_heads=4, vdim=64, scale=0.18, diff=0.4, rot_dims=32, base=500.0,
                                 kv_from=0), None),
], width=128, vocab=211, eps=3e-6)
# everything that can be one is one: one layer, one head, one key head, one expert of one, a recurrence of one
# channel in the second configuration; sizes that are no multiple of anything
RAK_C = config([
    layer("attention", attention(dim=6, heads=1, kv_heads=1, vdim=5, scale=1.0, diff=0.5, rot_dims=2, base=2.0, factor=1.0),
          moe(ff=8, experts=1, top=1, scale=1.0, shared=8)),
], width=32, vocab=50)
RAK_D = config([
    layer("mingru", mingru(1), dense(20)),
    layer("attention", attention(dim=20, heads=6, kv_heads=3, vdim=48, scale=0.2, diff=0.3, rot_dims=20, base=30.0,
                                 factor=8.0), moe(ff=40, experts=5, top=2, scale=2.5, shared=24)),
    layer("mingru", mingru(300), None),
], width=40, vocab=130)
