#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Llama-3.2-1B sizes with random weights, on one GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--sizes 1b|3b|8b] [--layers N]
    python bench.py --workload serve3b|long8b [--layers N] [--requests R]

A "step" is one decode step of the whole engine (scheduler, step function, sampler).  The default run has the
layer sizes of Llama-3.2-1B (16 layers, width 2048, 32 heads over 8 KV heads of 64, feed-forward 8192, vocabulary
128256, llama3 rope scaling, tied head), bfloat16, random weights N(0, 0.02), 2048-token prompts of uniform random
token ids, a batch of 8, and a maximum context of 8192.  It prints ONE JSON line: decoded tokens a second as
``value``, plus the 2048-token prefill, the decode step's roofline fraction (bytes it has to read / time / 8 TB/s)
and decode throughput at batch 1 and 64; the read and copy bandwidth and the MFMA rate that this GPU delivers,
measured by small probes, stand beside the published peaks (which stay the yardstick of every fraction).

``--compare somesun`` measures the Somesun decoder (attention with chunks and sinks beside a gated delta rule, routed
experts) at layer sizes that resemble a real model's, beside the Llama of equal width, heads and active feed-forward
width: prefill of 2,048 tokens and decode steps at batch 1, 8 and 64 through the same engine, ONE line of its own
(``--sizes 1b|3b`` picks the pair, ``--layers`` how many layers of each, 4 by default; ``--only`` one of the two).
``--compare morulix`` does the same for the Morulix decoder (latent attention, a state-space recurrence and windowed
attention in turn, each beside a dense feed-forward, behind one pass of its loop's entry), and ``--compare rakuvik``
for the Rakuvik decoder (differential attention and a minGRU recurrence in turn, dense and routed feed-forwards in
turn, the layers' results averaged over depth).  ``--compare bafilorn`` measures the Bafilorn decoder (a stream in
four copies behind an embedding of token pairs; latent attention with a rotated key part, lightning attention, and
chunked attention with tied values beside a gated linear recurrence in turn, each before a dense feed-forward with the
square of relu) beside the Morulix of equal sizes, the closest of the other designs, and the Llama.

``--workload`` runs one of the other two workloads instead and prints ONE line of its own:
``serve3b``: Llama-3.2-3B sizes, 64 requests with prompt lengths uniform in [128, 4096] (seeded), 256 generated tokens
each, continuous batching with chunked prefill under 2,048 tokens a step; ``long8b``: Llama-3.1-8B sizes, 16 requests
of 32,768 tokens of context (32,512 of prompt, 256 generated), prompts in 2,048-token portions beside decoding
requests.  ``value`` is generated tokens a second over the whole run, prompts included.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

LLAMA_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 2048, "intermediate_size": 8192, "vocab_size": 128256, "num_hidden_layers": 16,
    "num_attention_heads": 32, "num_key_value_heads": 8, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192, "rope_type": "llama3"},
    "max_position_embeddings": 131072, "tie_word_embeddings": True,
}
# other members of the family, for measurements beside the default (``--sizes``): what differs from LLAMA_1B
OTHER_SIZES = {
    "3b": dict(hidden_size=3072, num_attention_heads=24, num_key_value_heads=8, intermediate_size=8192,
               num_hidden_layers=28),
    "8b": dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, intermediate_size=14336,
               num_hidden_layers=32, tie_word_embeddings=False,
               rope_scaling=dict(LLAMA_1B["rope_scaling"], factor=8.0)),
}


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def make_engine(model, batch, context, page=16):
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig, ValidationConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    pages = batch * (-(-context // page)) + 8
    return LlmEngine(model, cache=CacheConfig(block_size=page, num_gpu_blocks_override=pages),
                     scheduler=SchedulerConfig(max_num_batched_tokens=max(2048, batch), max_num_sequences=max(batch, 1),
                                               max_model_len=context, enable_chunked_prefill=True),
                     validation=ValidationConfig(max_input_length=context - 1, max_total_tokens=context))


def decode_run(model, batch, prompt_len, steps, warmup, context, seed=0, sampling=None):
    """Prefill ``batch`` prompts (untimed), then time ``steps`` decode steps.  Returns (seconds, mean context)."""
    import torch
    from atoma_infer_amd.sampling import GenerateParameters
    eng = make_engine(model, batch, context)
    g = torch.Generator().manual_seed(seed)
    vocab = model.vocab_size
    # requests that finish their prompt early decode while the others are still in theirs
    # (the decoded tokens share the step's budget with the prompts, hence the factor of two)
    prompt_steps = 2 * batch * (-(-prompt_len // max(2048, batch)))
    params = GenerateParameters(do_sample=False, max_new_tokens=steps + warmup + prompt_steps + 8,
                                ignore_eos_token=True)
    if sampling:        # (temperature, top_k, top_p): draw instead of the default argmax
        params = GenerateParameters(do_sample=True, temperature=sampling[0], top_k=sampling[1] or None,
                                    top_p=sampling[2] if sampling[2] < 1.0 else None,
                                    random_seed=seed, max_new_tokens=params.max_new_tokens, ignore_eos_token=True)
    for _ in range(batch):
        eng.add_request(torch.randint(0, vocab, (prompt_len,), generator=g).tolist(), params)
    while any(r.in_prefill for r in eng.scheduler.running) or eng.scheduler.waiting:
        eng.step()
    for _ in range(warmup):
        eng.step()
    eng.drain()
    ctx0 = sum(r.length for r in eng.scheduler.running)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        eng.step()
    eng.drain()             # the engine runs one step ahead of the sampled tokens: read the last ones too
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx1 = sum(r.length for r in eng.scheduler.running)
    assert len(eng.scheduler.running) == batch, "a request ended or was preempted during the timed steps"
    mean_ctx = (ctx0 + ctx1) / 2.0 / batch
    del eng
    torch.cuda.empty_cache()
    return dt, mean_ctx


def prefill_run(model, n_tokens, reps, context):
    import torch
    from atoma_infer_amd.cache import CachePool, plan_cache
    from atoma_infer_amd.engine import ModelRunner, StepEntry
    plan = plan_cache(model.spec)
    pool = CachePool(plan, 16, [(-(-n_tokens // 16)) + 4] * len(plan.groups), 4, model.act_dtype, model.device)
    runner = ModelRunner(model, pool)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, model.vocab_size, (n_tokens,), generator=g).tolist()
    times = []
    for i in range(reps + 1):
        runner.add_request(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry(i, toks, 0, [n_tokens - 1])])
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        runner.free_request(i)
    del runner, pool
    torch.cuda.empty_cache()
    return min(times[1:])


WORKLOADS = {
    # name: (sizes, requests, shortest prompt, longest prompt, generated tokens, tokens a step)
    "serve3b": ("3b", 64, 128, 4096, 256, 2048),
    "long8b": ("8b", 16, 32768 - 256, 32768 - 256, 256, 2048),
}


def serve_run(model, n_req, lo, hi, out_tokens, budget, seed=3):
    """All requests arrive at once; the engine runs them to their end.  Returns what was measured."""
    import random

    import torch
    from atoma_infer_amd.config import CacheConfig, SchedulerConfig, ValidationConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling import GenerateParameters
    rnd = random.Random(seed)
    lens = [rnd.randint(lo, hi) for _ in range(n_req)]
    ctx = hi + out_tokens + 16
    pages = sum(-(-(n + out_tokens) // 16) + 1 for n in lens) + 64
    eng = LlmEngine(model, cache=CacheConfig(block_size=16, num_gpu_blocks_override=pages),
                    scheduler=SchedulerConfig(max_num_batched_tokens=budget, max_num_sequences=n_req,
                                              max_model_len=ctx, enable_chunked_prefill=True),
                    validation=ValidationConfig(max_input_length=ctx - 1, max_total_tokens=ctx))
    g = torch.Generator().manual_seed(1)
    params = GenerateParameters(do_sample=False, max_new_tokens=out_tokens, ignore_eos_token=True)
    for n in lens:
        eng.add_request(torch.randint(0, model.vocab_size, (n,), generator=g).tolist(), params)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps, done, times, last = 0, 0, [], t0
    while eng.has_unfinished():
        done += len(eng.step())
        now = time.perf_counter()
        times.append(now - last)
        last = now
        steps += 1
        if steps % 200 == 0:
            log(f"  step {steps}: {done} of {n_req} requests done, {now - t0:.1f} s")
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    times.sort()
    assert done == n_req
    return {"seconds": dt, "prompt_tokens": sum(lens), "generated": n_req * out_tokens, "steps": steps,
            "preemptions": eng.stats["preemptions"], "step_median_ms": times[len(times) // 2] * 1e3,
            "step_p99_ms": times[int(len(times) * 0.99)] * 1e3}


def somesun_like(llama: dict, layers: int) -> dict:
    """The Somesun configuration beside ``llama``: the same width, vocabulary, attention heads and head size; chunks of
    1,024 positions; a recurrent branch of half as many heads of 128 x 128; experts of a quarter (1b) or half (3b) of
    the dense feed-forward's width of which as many are chosen as make up that width."""
    w, nh, nkv = llama["hidden_size"], llama["num_attention_heads"], llama["num_key_value_heads"]
    hd = w // nh
    rh = w // 256
    ff = 2048 if w <= 2048 else 4096
    top = llama["intermediate_size"] // ff
    layer = {"type": "parallel",
             "mixer": {"left": {"dim": hd, "heads": nh, "kv_heads": nkv, "vdim": hd, "scale": hd ** -0.5,
                                "mask": {"size": 1024}, "rot": {"base": 500000.0, "dims": hd}},
                       "right": {"dim": 128, "heads": rh, "kv_heads": rh // 2, "vdim": 128, "conv": 4,
                                 "decay_rank": 64, "gate_rank": 64},
                       "left_scale": 0.5, "right_scale": 0.5},
             "mlp": {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": 8 * top, "top": top}}}
    return {"architecture": "Somesun", "layers": [layer] * layers, "norm": {"eps": 1e-5},
            "vocab": llama["vocab_size"], "width": w, "max_positions": llama["max_position_embeddings"]}


def step_bytes_somesun(cfg: dict, batch: int, ctx: float) -> float:
    """Bytes a decode step of ``batch`` requests at context ``ctx`` has to read (and, for the state, write): every
    dense matrix once, the experts that ``batch`` tokens are expected to choose between them, the keys and values of
    each request's current chunk, the recurrent state twice."""
    total = 2.0 * cfg["vocab"] * cfg["width"]
    w = cfg["width"]
    for l in cfg["layers"]:
        a, r, m = l["mixer"]["left"], l["mixer"]["right"], l["mlp"]
        total += 2.0 * w * (2 * a["heads"] + a["kv_heads"]) * a["dim"]
        rq, rv = r["kv_heads"] * r["dim"], r["heads"] * r["vdim"]
        total += 2.0 * (w * (2 * rq + 2 * rv + r["heads"] + r["decay_rank"] + r["gate_rank"])
                        + r["decay_rank"] * r["heads"] * r["dim"] + r["gate_rank"] * rv)
        e, top = m["router"]["experts"], m["router"]["top"]
        chosen = e * (1.0 - (1.0 - top / e) ** batch)
        total += 2.0 * w * e + chosen * 2.0 * 3 * w * m["expert"]["ff"]
        seen = min(ctx, a["mask"]["size"] / 2.0)
        total += batch * (2.0 * 2 * a["kv_heads"] * a["dim"] * seen + 2 * 4.0 * r["heads"] * r["dim"] * r["vdim"])
    return total


def morulix_like(llama: dict, layers: int) -> dict:
    """The Morulix configuration beside ``llama``: the same width, vocabulary and dense feed-forward; layers in turn
    latent attention (half as many heads of twice the size over a latent of 128 numbers, 256 from a width of 3,072
    on), a state-space recurrence
    (inner width twice the model's, heads of 64 columns, a state of 128, one group), windowed attention with the
    Llama's heads and a window of 1,024 keys, and the recurrence again; one pass of the loop's entry over all layers."""
    w, nh, nkv = llama["hidden_size"], llama["num_attention_heads"], llama["num_key_value_heads"]
    hd = w // nh
    mlp = {"kind": "dense", "ff": llama["intermediate_size"]}
    sc = llama["rope_scaling"]
    att = {"type": "attention", "mlp": mlp,
           "mixer": {"dim": hd, "heads": nh, "kv_heads": nkv, "vdim": hd, "scale": hd ** -0.5, "mask": {"size": 1024},
                     "rot": {"base": llama["rope_theta"], "dims": hd,
                             "scaling": {"factor": sc["factor"], "low": sc["low_freq_factor"],
                                         "high": sc["high_freq_factor"], "original": sc["original_max_position_embeddings"]}}}}
    lat = {"type": "latent_attention", "mlp": mlp,
           "mixer": {"dim": 2 * hd, "heads": nh // 2, "kv_rank": 128 if w < 3072 else 256, "scale": (2 * hd) ** -0.5, "vdim": 2 * hd}}
    ssm = {"type": "mamba2", "mlp": mlp,
           "mixer": {"conv": 4, "groups": 1, "heads": 2 * w // 64, "norm_groups": 1, "state": 128, "vdim": 64}}
    kinds = [lat, ssm, att, ssm]
    return {"architecture": "Morulix", "layers": [kinds[i % 4] for i in range(layers)], "norm": {"eps": 1e-5},
            "loop": {"start": 0, "stop": layers, "times": 1}, "vocab": llama["vocab_size"], "width": w,
            "max_positions": llama["max_position_embeddings"]}


def step_bytes_morulix(model, cfg: dict, batch: int, ctx: float) -> float:
    """Bytes a decode step of ``batch`` requests at context ``ctx`` has to read (and, for the state, write): every
    matrix once, each request's latents (kept once in the keys' order and once in the values'), the keys and values
    inside its window, the recurrent state twice."""
    total = float(model.weight_bytes())
    for l in cfg["layers"]:
        m = l["mixer"]
        if l["type"] == "latent_attention":
            total += batch * ctx * 2.0 * 2 * (-(-m["kv_rank"] // 16) * 16)
        elif l["type"] == "attention":
            seen = min(ctx, m["mask"]["size"]) if m.get("mask") else ctx
            total += batch * seen * 2.0 * 2 * m["kv_heads"] * max(m["dim"], m["vdim"])
        else:
            total += batch * 2 * 4.0 * m["heads"] * m["vdim"] * m["state"]
    return total


def rakuvik_like(llama: dict, layers: int) -> dict:
    """The Rakuvik configuration beside ``llama``: the same width and vocabulary; layers in turn differential attention
    (half as many heads, each of two maps of the Llama's head size over values of twice that, so that queries, keys and
    values are as wide as the Llama's) before a dense feed-forward of the Llama's width, a minGRU recurrence of twice
    the model's width before routed experts (squared ReLU, 2,048 columns, as many chosen of eight times as many as
    make up the dense width, and a shared one), differential attention that reads the first layer's keys and values,
    and the recurrence again."""
    w, nh, nkv = llama["hidden_size"], llama["num_attention_heads"], llama["num_key_value_heads"]
    hd = w // nh
    ff = 2048
    top = llama["intermediate_size"] // ff
    dense = {"kind": "dense", "ff": llama["intermediate_size"]}
    moe = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": 8 * top, "scale": 2.5, "top": top},
           "shared": {"ff": ff}}
    mixer = {"dim": hd, "heads": nh // 2, "kv_heads": max(1, nkv // 2), "vdim": 2 * hd, "scale": hd ** -0.5, "diff": 0.8,
             "rot": {"base": llama["rope_theta"], "dims": hd, "scaling": {"factor": 4.0}}}
    out = []
    for i in range(layers):
        if i % 2:
            out.append({"type": "mingru", "mixer": {"width": 2 * w}, "mlp": moe})
        elif i % 4 == 2:
            out.append({"type": "attention", "mixer": dict(mixer, kv_from=i - 2), "mlp": dense})
        else:
            out.append({"type": "attention", "mixer": mixer, "mlp": dense})
    return {"architecture": "Rakuvik", "layers": out, "norm": {"eps": 1e-5}, "vocab": llama["vocab_size"], "width": w,
            "max_positions": llama["max_position_embeddings"]}


def step_bytes_rakuvik(model, cfg: dict, batch: int, ctx: float) -> float:
    """Bytes a decode step of ``batch`` requests at context ``ctx`` has to read (and, for the state, write): every
    dense matrix once, the experts that ``batch`` tokens are expected to choose between them, the keys of both maps
    and the values of every attention layer (one that reads another layer's reads them again), the recurrent state
    twice, and the kept results of all layers once for every layer behind them."""
    total = float(model.weight_bytes())
    w = cfg["width"]
    for i, l in enumerate(cfg["layers"]):
        m, f = l["mixer"], l["mlp"]
        if l["type"] == "attention":
            total += batch * ctx * 2.0 * 2 * m["kv_heads"] * max(2 * m["dim"], m["vdim"])
        else:
            total += batch * 2 * 4.0 * m["width"]
        if f and f["kind"] == "moe":
            e, top = f["router"]["experts"], f["router"]["top"]
            total += (e * (1.0 - (1.0 - top / e) ** batch) - top) * 2.0 * 2 * w * f["expert"]["ff"]
        total += batch * 4.0 * w * (i + 2)
    return total


def bafilorn_like(llama: dict, layers: int) -> dict:
    """The Bafilorn configuration beside ``llama`` and ``morulix_like(llama)``: the same width and vocabulary; four
    copies of the stream; a table of 65,521 token pairs; layers in turn latent attention (half as many heads of twice
    the size, 32 of their columns rotated, over a cached key of the Morulix's latent width, queries through a latent of
    half the model's width), lightning attention (as many heads as the Llama, keys and values of 128 columns: a state
    as large as the Morulix recurrence's), chunked attention with the Llama's heads and tied values beside a gated
    linear recurrence of the model's width in 16 blocks, and lightning attention again; feed-forwards of one and a half
    times the Llama's width (two matrices where the gated one has three)."""
    w, nh, nkv = llama["hidden_size"], llama["num_attention_heads"], llama["num_key_value_heads"]
    hd = w // nh
    mlp = {"kind": "dense", "ff": 3 * llama["intermediate_size"] // 2}
    wide = 128 if w < 3072 else 256
    lat = {"type": "latent_attention", "mlp": mlp,
           "mixer": {"dim": 2 * hd - 32, "heads": nh // 2, "kv_rank": wide - 32 if wide == 256 else wide, "q_rank": w // 2,
                     "rot_dim": 32, "rot": {"base": 10000.0, "dims": 32}, "scale": (2 * hd) ** -0.5, "vdim": 2 * hd}}
    lit = {"type": "lightning", "mlp": mlp,
           "mixer": {"decay": [1.0 - 2.0 ** (-3.0 - 5.0 * h / nh) for h in range(nh)], "dim": 128, "heads": nh, "vdim": 128}}
    par = {"type": "parallel", "mlp": mlp,
           "mixer": {"left": {"dim": hd, "heads": nh, "kv_heads": nkv, "vdim": hd, "scale": hd ** -0.5,
                              "mask": {"size": 1024},
                              "rot": {"base": llama["rope_theta"], "dims": hd,
                                      "scaling": {"factor": 8.0, "original": 8192, "fast": 16.0, "slow": 2.0}}},
                     "right": {"blocks": 16, "conv": 4, "width": w}}}
    kinds = [lat, lit, par, lit]
    return {"architecture": "Bafilorn", "embedding": {"scale": 1.0, "bigram": {"buckets": 65521, "mul_prev": 1000003, "mul_cur": 40503}},
            "layers": [kinds[i % 4] for i in range(layers)], "norm": {"eps": 1e-5}, "streams": 4,
            "loop": {"start": 0, "stop": layers, "times": 1}, "vocab": llama["vocab_size"], "width": w,
            "max_positions": llama["max_position_embeddings"]}


def step_bytes_bafilorn(model, cfg: dict, batch: int, ctx: float) -> float:
    """Bytes a decode step of ``batch`` requests at context ``ctx`` has to read (and, for the states, write): every
    matrix once, each request's cached keys and values of the latent layers (both as wide as the key), the keys and
    values of its current chunk, the recurrent states twice, the copies of the stream twice per sublayer."""
    total = float(model.weight_bytes())
    w, copies = cfg["width"], cfg.get("streams") or 1
    for l in cfg["layers"]:
        m = l["mixer"]
        if l["type"] == "latent_attention":
            total += batch * ctx * 2.0 * 2 * (-(-(m["kv_rank"] + m["rot_dim"]) // 16) * 16)
        elif l["type"] == "lightning":
            total += batch * 2 * 4.0 * m["heads"] * m["dim"] * m["vdim"]
        else:
            a, r = m["left"], m["right"]
            seen = min(ctx, a["mask"]["size"] / 2.0) if a.get("mask") else ctx
            total += batch * (2.0 * 2 * a["kv_heads"] * a["dim"] * seen + 2 * 4.0 * r["conv"] * r["width"])
        total += batch * 4.0 * w * copies * 2 * (2 if l["mlp"] else 1)
    return total


def compare_main(args) -> int:
    import torch
    import atoma_infer_amd  # noqa: F401
    from atoma_infer_amd.cache import plan_cache
    from atoma_infer_amd.models import random_model
    sizes = args.sizes if args.sizes in ("1b", "3b") else "1b"
    layers = args.layers or 4
    llama = dict(dict(LLAMA_1B, **OTHER_SIZES.get(sizes, {})), num_hidden_layers=layers)
    design = args.compare
    sun = {"somesun": somesun_like, "morulix": morulix_like, "rakuvik": rakuvik_like,
           "bafilorn": bafilorn_like}[design](llama, layers)
    out = {}
    pairs = [("llama", llama), (design, sun)]
    if design == "bafilorn":      # also the closest of the other designs, at the same sizes
        pairs.insert(1, ("morulix", morulix_like(llama, layers)))
    for name, cfg in pairs:
        if args.only and args.only != name:
            continue
        log(f"{name}: building {layers} layers at {sizes} sizes (random weights) ...")
        model = random_model(cfg, seed=0, dtype="bfloat16", stored="bfloat16")
        pre_s = prefill_run(model, args.prefill_tokens, 4, args.context)
        res = {"prefill_ms": round(pre_s * 1e3, 3), "prefill_tok_s": round(args.prefill_tokens / pre_s, 1)}
        kv = plan_cache(model.spec).bytes_per_token(2)
        for b in (1, 8, 64):
            st = min(args.steps, 64)
            log(f"{name}: decode at batch {b} ...")
            d, ctx = decode_run(model, b, args.prompt_len, st, min(args.warmup, 4), args.context)
            if name == "somesun":
                nbytes = step_bytes_somesun(sun, b, ctx)
            elif name == "bafilorn":
                nbytes = step_bytes_bafilorn(model, sun, b, ctx)
            elif name == "morulix":
                nbytes = step_bytes_morulix(model, cfg, b, ctx)
            elif name == "rakuvik":
                nbytes = step_bytes_rakuvik(model, sun, b, ctx)
            else:
                nbytes = model.weight_bytes() + kv * ctx * b
            res[f"decode_b{b}_tok_s"] = round(b * st / d, 1)
            res[f"decode_b{b}_ms"] = round(d / st * 1e3, 4)
            res[f"decode_b{b}_frac"] = round(nbytes / (d / st) / 1e9 / HBM_PEAK_GBS, 4)
        out[name] = res
        del model
        torch.cuda.empty_cache()
    l = sun["layers"][0]
    if design == "somesun":
        shown = {"left": l["mixer"]["left"], "right": l["mixer"]["right"], "mlp": l["mlp"]}
    elif design == "morulix":
        shown = {"layers_in_turn": [{"type": x["type"], "mixer": x["mixer"]} for x in sun["layers"][:4]], "mlp": l["mlp"],
                 "loop": sun["loop"]}
    else:
        shown = {"layers_in_turn": sun["layers"][:4]}
    line = {"metric": f"{design.capitalize()} beside Llama at {sizes} layer sizes, {layers} layers each: prefill of "
                      f"{args.prefill_tokens} tokens, decode at batch 1, 8, 64 ({args.prompt_len}-token prompts)",
            "unit": "tokens/s, ms a step, fraction of 8 TB/s", "n_gpus": 1, "dtype": "bf16",
            "data": "synthetic (uniform random token ids, random weights)",
            "config": {"width": sun["width"], "vocab": sun["vocab"], "layers": layers, **shown,
                       "llama": {k: llama[k] for k in ("hidden_size", "intermediate_size", "num_attention_heads",
                                                        "num_key_value_heads")}},
            **out}
    print(json.dumps(line), flush=True)
    return 0


def workload_main(args) -> int:
    import atoma_infer_amd  # noqa: F401
    from atoma_infer_amd.models import random_model
    sizes, n_req, lo, hi, out_tokens, budget = WORKLOADS[args.workload]
    n_req = args.requests or n_req
    base = dict(LLAMA_1B, **OTHER_SIZES[sizes])
    full_layers = base["num_hidden_layers"]
    layers = args.layers or full_layers
    name = {"3b": "Llama-3.2-3B", "8b": "Llama-3.1-8B"}[sizes]
    log(f"{args.workload}: building {name} sizes ({layers} of {full_layers} layers, random weights) ...")
    model = random_model(dict(base, num_hidden_layers=layers), seed=0, dtype="bfloat16", stored="bfloat16")
    log(f"{n_req} requests, prompts of {lo} to {hi} tokens, {out_tokens} generated each, {budget} tokens a step ...")
    r = serve_run(model, n_req, lo, hi, out_tokens, budget)
    c = model.config
    line = {
        "metric": f"generated tok/s, workload {args.workload} ({name} sizes, {n_req} requests, continuous batching "
                  f"with chunked prefill)",
        "value": round(r["generated"] / r["seconds"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": r["steps"],
        "warmup": 0, "ms_per_step": round(r["seconds"] / r["steps"] * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic (uniform random token ids, random weights N(0, 0.02))",
        "config": {"model": name + " sizes", "layers": layers, "layers_full": full_layers, "hidden": c.hidden_size,
                   "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads, "head_dim": c.head_size,
                   "intermediate": c.intermediate_size, "vocab": c.vocab_size, "requests": n_req,
                   "prompt_min": lo, "prompt_max": hi, "generated_each": out_tokens, "tokens_a_step": budget,
                   "kv_block": 16, "sampling": "argmax", "parallelism": "single GPU"},
        "total_tokens_per_s": round((r["prompt_tokens"] + r["generated"]) / r["seconds"], 1),
        "prompt_tokens": r["prompt_tokens"], "generated_tokens": r["generated"], "seconds": round(r["seconds"], 3),
        "preemptions": r["preemptions"], "step_median_ms": round(r["step_median_ms"], 3),
        "step_p99_ms": round(r["step_p99_ms"], 3),
    }
    print(json.dumps(line), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--sizes", choices=["1b", "3b", "8b"], default="1b",
                    help="layer sizes of Llama-3.2-1B (the default run), Llama-3.2-3B or Llama-3.1-8B")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the model has (default: all)")
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 runs")
    ap.add_argument("--temperature", type=float, default=0.0,
                    help="sample with this temperature (and --top-k, --top-p) instead of the default argmax")
    ap.add_argument("--top-k", type=int, default=0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--workload", choices=["decode", *WORKLOADS], default="decode",
                    help="decode: the default run; serve3b, long8b: the other two workloads, one line of their own")
    ap.add_argument("--compare", choices=["somesun", "morulix", "rakuvik", "bafilorn"], default=None,
                    help="measure that design at --sizes (1b, 3b) beside the Llama of equal sizes, one line of its own")
    ap.add_argument("--only", choices=["llama", "somesun", "morulix", "rakuvik", "bafilorn"], default=None, help="with --compare: one of the two models")
    ap.add_argument("--requests", type=int, default=0, help="requests of a --workload run (default: the workload's)")
    ap.add_argument("--no-peaks", action="store_true", help="skip the probes of what the GPU delivers")
    ap.add_argument("--chain-floors", action="store_true",
                    help="only measure what a chain of dependent kernels costs beyond its bytes (an empty kernel, read "
                         "streams of 8 to 64 MB, a grid-wide barrier), print one JSON line and stop")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported", flush=True)
        return 2
    if int(os.environ.get("WORLD_SIZE", "1")) > 1:
        print("bench.py: started with WORLD_SIZE > 1; this engine runs on one GPU", flush=True)
        return 2
    if args.chain_floors:
        import atoma_infer_amd  # noqa: F401
        from atoma_infer_amd.kernels.ops import measure_chain_floors
        print(json.dumps({"chain_floors": measure_chain_floors(), "unit": "us a kernel"}), flush=True)
        return 0
    if args.compare:
        return compare_main(args)
    if args.workload != "decode":
        return workload_main(args)
    if args.prompt_len + args.steps + args.warmup + 2 * args.batch * (-(-args.prompt_len // 2048)) + 8 > args.context:
        print("bench.py: prompt + steps exceed the context", file=sys.stderr)
        return 1

    import torch
    import atoma_infer_amd  # noqa: F401
    from atoma_infer_amd.cache import plan_cache
    from atoma_infer_amd.models import random_model

    base = dict(LLAMA_1B, **OTHER_SIZES.get(args.sizes, {}))
    full_layers = base["num_hidden_layers"]
    args.layers = args.layers or full_layers
    cfg = dict(base, num_hidden_layers=args.layers)
    name = {"1b": "Llama-3.2-1B", "3b": "Llama-3.2-3B", "8b": "Llama-3.1-8B"}[args.sizes]
    log(f"building the model ({args.layers} layers, random weights) ...")
    t0 = time.time()
    model = random_model(cfg, seed=0, dtype="bfloat16", stored="bfloat16")
    log(f"model ready in {time.time() - t0:.1f} s; weights read per step: {model.weight_bytes() / 1e6:.1f} MB")
    kv_bytes_per_token = plan_cache(model.spec).bytes_per_token(2)

    log(f"prefill of {args.prefill_tokens} tokens ...")
    pre_s = prefill_run(model, args.prefill_tokens, 8, args.context)
    c = model.config
    hd = c.head_size
    layer_params = (c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * hd
                    + c.num_attention_heads * hd * c.hidden_size + 3 * c.hidden_size * c.intermediate_size)
    t = args.prefill_tokens
    pre_flops = (2.0 * t * layer_params * c.num_hidden_layers
                 + 4.0 * (t * (t + 1) / 2.0) * hd * c.num_attention_heads * c.num_hidden_layers
                 + 2.0 * c.hidden_size * c.vocab_size)
    prefill = {"value": round(t / pre_s, 1), "tokens": t, "ms": round(pre_s * 1e3, 3),
               "frac": round(pre_flops / pre_s / PEAK_FLOPS["bf16"], 4)}

    log(f"decode at batch {args.batch}: {args.warmup} warm-up + {args.steps} timed steps ...")
    sampling = (args.temperature, args.top_k, args.top_p) if args.temperature > 0 else None
    dt, mean_ctx = decode_run(model, args.batch, args.prompt_len, args.steps, args.warmup, args.context,
                              sampling=sampling)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = model.weight_bytes() + kv_bytes_per_token * mean_ctx * args.batch
    achieved = step_bytes / (dt / args.steps) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4)}

    points = {}
    if not args.no_points:
        for b, st in ((1, min(args.steps, 128)), (64, min(args.steps, 64))):
            log(f"decode at batch {b} ...")
            d, ctx_b = decode_run(model, b, args.prompt_len, st, min(args.warmup, 4), args.context, sampling=sampling)
            points[f"decode_b{b}"] = round(b * st / d, 1)
            # the same roofline fraction as the headline's, with this batch's own mean context
            bytes_b = model.weight_bytes() + kv_bytes_per_token * ctx_b * b
            points[f"decode_b{b}_frac"] = round(bytes_b / (d / st) / 1e9 / HBM_PEAK_GBS, 4)

    # the probes of what the GPU delivers run last: minutes of full load before the timed steps would only warm the
    # chip against them
    peaks = {}
    if not args.no_peaks:
        from atoma_infer_amd.kernels.ops import measure_device_peaks
        log("probing what the GPU delivers (read stream, copy, MFMA loop) ...")
        peaks = measure_device_peaks(model.device)
        log(f"  {peaks}")
    if peaks:
        # what the probes reached on this GPU, beside the published peaks that the fractions above are of
        roofline["measured_peak"] = peaks["hbm_read_gbs"]
        roofline["measured_how"] = peaks.get("hbm_read_how", "")
        roofline["measured_copy"] = peaks["hbm_copy_gbs"]
        roofline["frac_of_measured"] = round(achieved / peaks["hbm_read_gbs"], 4)
        prefill["measured_peak_tflops"] = peaks["mfma_bf16_tflops"]
        prefill["frac_of_measured"] = round(pre_flops / pre_s / (peaks["mfma_bf16_tflops"] * 1e12), 4)

    line = {
        "metric": f"decode tok/s at batch {args.batch} ({name} sizes, {args.prompt_len}-token prompts); "
                  "points: batch 1 and 64; prefill tok/s at 2048 tokens",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (uniform random token ids, random weights N(0, 0.02))",
        "config": {"model": name + " sizes",
                   "layers": args.layers, "layers_full": full_layers,
                   "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
                   "head_dim": hd, "intermediate": c.intermediate_size, "vocab": c.vocab_size,
                   "global_batch": args.batch, "seq_len": args.prompt_len, "context": args.context,
                   "mean_decode_context": round(mean_ctx, 1), "kv_block": 16, "sampling": ("argmax" if not sampling else f"T={sampling[0]} top_k={sampling[1]} top_p={sampling[2]}"),
                   "tied_embeddings": bool(base["tie_word_embeddings"]),
                   "parallelism": "single GPU"},
        "prefill": prefill, "roofline": roofline, "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
