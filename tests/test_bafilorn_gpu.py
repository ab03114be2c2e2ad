"""Bafilorn on the GPU against the plain implementation: every mechanism alone, then the whole model through the
runner's step function (portions, batches, pages and slots used again) and through the engine's own entry point."""
import copy
import json
import os
import types

import numpy as np
import pytest
import torch

import plain_bafilorn as pb
from bafilorn_util import (BAF_A, BAF_B, BAF_C, BAF_D, as_numpy, config, latent, layer, lightning, numpy_weights,
                           parallel, random_config)
from somesun_util import make_runner, plain_config, row_errors, run_schedule, tokens, write_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# float32: the engine's sums run in another order than the plain model's float64 ones; bfloat16: activations are
# rounded to 8 bits about ten times a layer
TOL = {"float32": 3e-5, "bfloat16": 4e-2}
PART_TOL = {torch.float32: 2e-5, torch.bfloat16: 2.5e-2}
CONFIGS = {"A": BAF_A, "B": BAF_B, "C": BAF_C, "D": BAF_D}


def _lively(t):
    """Connection weights that mix in earnest, recurrences that hold on for a while, biases that matter."""
    g = torch.Generator().manual_seed(5)
    for k in t:
        if k.endswith(".mix") and ".hc" in k:
            t[k] = t[k] + 0.3 * torch.randn(t[k].shape, generator=g)
        elif k.endswith(".lam"):
            t[k] = t[k] - 1.5
        elif k.endswith((".q.b", ".k.b", ".o.b", ".y.b", ".x.b")):
            t[k] = t[k] * 3


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("bafilorn")
    return {n: write_model(str(root / n), c, 41 + i, _lively) for i, (n, c) in enumerate(CONFIGS.items())}


def oracle(path, toks):
    return torch.from_numpy(pb.forward(list(toks), numpy_weights(path), plain_config(path))[0]).float()


def assert_logits(got, want, dtype, what=""):
    e = row_errors(got, want)
    assert float(e.max()) < TOL[dtype], (what, float(e.max()), int(e.argmax()))


def _ctx(starts, counts, slots, toks=None):
    """What a part reads of a step, for entries of ``counts`` tokens at ``starts``, built by hand."""
    t = int(sum(counts))
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    seq = [e for e, c in enumerate(counts) for _ in range(c)]
    pos = [s + j for s, c in zip(starts, counts) for j in range(c)]
    q_start = np.concatenate([[0], np.cumsum(counts)]).tolist()
    return types.SimpleNamespace(n_tokens=t, n_entries=len(counts), positions=i32(pos), token_seq=i32(seq),
                                 q_start=i32(q_start), state_slots=i32(slots), h_starts=np.asarray(starts, dtype=np.int32),
                                 h_counts=np.asarray(counts, dtype=np.int32), plans={}, scratch={}, decode_bucket=None,
                                 tokens=i32(toks) if toks is not None else None)


def _load(part, weights, dtype):
    part.load(lambda name: weights[name].to(torch.bfloat16), torch.device(DEV), dtype)


def _drawn(part, tag, seed, boost=()):
    """Random tensors for a part as bfloat16 values held in float32; ``boost`` names tensors to make larger."""
    from atoma_infer_amd.weights.random_init import random_tensor
    w = {n: random_tensor(tag + n, ws, seed, torch.bfloat16, 0.1).float() for n, ws in part.weight_specs().items()}
    for n, f in boost:
        if n in w:
            w[n] = (w[n] * f).to(torch.bfloat16).float()
    return w


def _flat(y):
    return (y.sum(0) if y.dim() == 3 else y).float().cpu()


def _rel(a, b):
    b = torch.as_tensor(b)
    return float((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30))


def _inputs(lens, width, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(c, width, generator=g).to(torch.bfloat16).float() for c in lens]


# ---- small kernels ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("copies, width, planes", [(1, 64, 1), (2, 200, 3), (3, 33, 1), (4, 4100, 2), (5, 50, 1), (8, 96, 1)])
def test_the_copies_of_the_stream_are_mixed_read_and_normed_in_one_pass(copies, width, planes):
    from atoma_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(copies * 1000 + width)
    t, eps = 7, 3e-6
    x = torch.randn(copies, t, width, generator=g)
    y = torch.randn(planes, t, width, generator=g)
    mix, out, win = torch.randn(copies, copies, generator=g), torch.randn(copies, generator=g), torch.randn(copies, generator=g)
    nw = torch.randn(width, generator=g)
    new = torch.einsum("st,snw->tnw", mix.double(), x.double()) + out.double()[:, None, None] * y.double().sum(0)
    u = torch.einsum("s,snw->nw", win.double(), new)
    want_h = torch.from_numpy(pb.unit_rms(u.numpy(), eps)) * nw.double()
    dy = (y[0] if planes == 1 else y).contiguous().to(DEV)
    for out_dtype in (torch.float32, torch.bfloat16):
        xd = x.to(DEV)
        h = ops.stream_step(xd, (dy, mix.to(DEV), out.to(DEV)), (win.to(DEV), nw.to(DEV), eps), out_dtype=out_dtype)
        assert (xd.cpu().double() - new).abs().max() < 1e-5
        assert _rel(h.float().cpu(), want_h) < (1e-6 if out_dtype is torch.float32 else 5e-3)
    # the update alone; the read alone (of the copies as they are); rows: the stream stays as it was
    xd = x.to(DEV)
    assert ops.stream_step(xd, (dy.to(torch.bfloat16) if planes == 1 else dy, mix.to(DEV), out.to(DEV))) is None
    assert (xd.cpu().double() - new).abs().max() < (0.1 if planes == 1 else 1e-5)
    xd = x.to(DEV)
    h = ops.stream_step(xd, None, (win.to(DEV), nw.to(DEV), eps), out_dtype=torch.float32)
    u0 = torch.einsum("s,snw->nw", win.double(), x.double())
    assert _rel(h.cpu(), torch.from_numpy(pb.unit_rms(u0.numpy(), eps)) * nw.double()) < 1e-6 and torch.equal(xd.cpu(), x)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    h = ops.stream_step(xd, (dy, mix.to(DEV), out.to(DEV)), (win.to(DEV), nw.to(DEV), eps), rows=rows, out_dtype=torch.float32)
    assert _rel(h.cpu(), want_h[[5, 0, 5]]) < 1e-6 and torch.equal(xd.cpu(), x)


@pytest.mark.parametrize("pairs", [(53, 7, 3), (1, 5, 9), (521, 65537, 40503), None])
def test_the_embedding_adds_the_row_of_the_pair_and_keeps_the_last_token_per_request(pairs):
    from atoma_infer_amd.parts import BigramEmbedding
    vocab, width, copies = 90, 40, 3
    part = BigramEmbedding(vocab, width, scale=2.5, pairs=pairs, copies=copies)
    w = _drawn(part, "e.", 2)
    _load(part, w, torch.float32)
    cfg = {"embedding": {"scale": 2.5}}
    if pairs:
        cfg["embedding"]["bigram"] = {"buckets": pairs[0], "mul_prev": pairs[1], "mul_cur": pairs[2]}
    reqs = [tokens(23, vocab, 1), tokens(9, vocab, 2)]
    want = [pb.embed(np.array(r), as_numpy(w), cfg) for r in reqs]
    state = torch.full((4, 1), 77, dtype=torch.int32, device=DEV)
    state[2].zero_()
    state[0].zero_()
    cache = types.SimpleNamespace(state=state if pairs else None)
    got, at = [[], []], [0, 0]
    for cuts in ([(0, 5), (1, 1)], [(1, 1), (0, 1)], [(0, 2)], [(1, 7), (0, 15)]):
        ctx = _ctx([at[r] for r, _ in cuts], [c for _, c in cuts], [2 if r == 0 else 0 for r, _ in cuts],
                   [tk for r, c in cuts for tk in reqs[r][at[r]: at[r] + c]])
        x = part.forward_step(ctx, cache).cpu()
        assert x.shape == (copies, ctx.n_tokens, width) and torch.equal(x[0], x[-1])
        o = 0
        for r, c in cuts:
            got[r].append(x[0, o: o + c])
            o += c
            at[r] += c
    for r in range(2):
        assert (torch.cat(got[r]).double() - torch.from_numpy(want[r])).abs().max() < 1e-6
    if pairs:
        assert state[:, 0].tolist() == [reqs[1][-1], 77, reqs[0][-1], 77]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, ff", [(64, 48), (40, 20), (128, 96), (200, 1), (384, 768)])
def test_the_feed_forward_squares_what_relu_lets_through(width, ff, dtype):
    from atoma_infer_amd.parts.base import make_part
    part = make_part("feed_forward", "dense", width=width, intermediate=ff, names=("up", "down"))
    w = _drawn(part, "f.", 3, boost=(("up", 10),))
    _load(part, w, dtype)
    for t in (1, 7, 70):
        h = _inputs([t], width, ff + t)[0]
        want = pb.feed_forward(h.double().numpy(), as_numpy(w, "m."), "m.")
        assert _rel(_flat(part.forward(h.to(DEV, dtype), None)), want) < PART_TOL[dtype], t


# ---- the recurrences alone ------------------------------------------------------------------------------------------

RECURRENT_CUTS = ([(0, 1), (1, 2)], [(0, 2)], [(1, 1), (0, 1)], [(0, 30), (1, 6)], [(0, 3)], [(0, 64), (1, 17)], [(0, 250)],
                  [(0, 16), (1, 100)], [(1, 3), (0, 100)])


def _recurrent_case(part, hs, dtype, state_width):
    """Two requests side by side in portions of one token, two, a few and hundreds, each carried by its state slot."""
    state = torch.full((4, state_width), float("nan"), dtype=torch.float32, device=DEV)
    state[1].fill_(7.0)                       # another request's slot must stay as it is
    state[0].zero_()
    state[3].zero_()
    cache = types.SimpleNamespace(state=state)
    got, at = [[], []], [0, 0]
    for cuts in RECURRENT_CUTS:
        ctx = _ctx([at[r] for r, _ in cuts], [c for _, c in cuts], [3 if r == 0 else 0 for r, _ in cuts])
        x = torch.cat([hs[r][at[r]: at[r] + c] for r, c in cuts]).to(DEV, dtype)
        y = _flat(part.forward(x, ctx, cache))
        o = 0
        for r, c in cuts:
            got[r].append(y[o: o + c])
            o += c
            at[r] += c
    assert at == [len(h) for h in hs] and bool((state[1] == 7.0).all()) and bool(state[2].isnan().all())
    return [torch.cat(g) for g in got]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dim, vdim", [(3, 16, 24), (1, 128, 64), (2, 10, 5), (1, 1, 1), (5, 200, 17), (2, 64, 32),
                                              (3, 32, 40), (2, 96, 16), (4, 128, 128)])
def test_lightning_attention_alone_whole_and_in_portions(heads, dim, vdim, dtype):
    from atoma_infer_amd.parts import LightningAttention
    width = 64
    m = lightning(heads, dim, vdim)
    part = LightningAttention(width, heads, dim, vdim, m["decay"], 1e-5)
    w = _drawn(part, "l.", 5, boost=(("q", 4), ("k", 4), ("v", 4), ("g", 8)))
    _load(part, w, dtype)
    hs = _inputs((467, 129), width, heads * dim)
    want = [pb.lightning(h.double().numpy(), as_numpy(w, "m."), "m.", m, 1e-5)[0] for h in hs]
    got = _recurrent_case(part, hs, dtype, heads * vdim * dim)
    for r in range(2):
        assert _rel(got[r], want[r]) < PART_TOL[dtype], r


def test_a_far_token_stays_in_the_state_of_a_head_that_hardly_decays():
    """One early token with a large value under a decay of 0.9995; hundreds of tokens later the read-out still holds
    it, while the head beside it, which decays fast, has forgotten.  A state that is lost, cleared or carried by the
    wrong slot changes the late outputs entirely."""
    from atoma_infer_amd.parts import LightningAttention
    width, m = 64, lightning(2, 32, 16, decay=[0.9995, 0.5])
    part = LightningAttention(width, 2, 32, 16, m["decay"], 1e-5)
    w = _drawn(part, "m.", 9, boost=(("q", 4), ("k", 4), ("v", 4)))
    _load(part, w, torch.float32)
    h = _inputs([400], width, 1)[0] * 0.3
    h[5] = h[5] * 100
    want = pb.lightning(h.double().numpy(), as_numpy(w, "m."), "m.", m, 1e-5)[0]
    h2 = h.clone()
    h2[5] = h[5] / 100
    without = pb.lightning(h2.double().numpy(), as_numpy(w, "m."), "m.", m, 1e-5)[0]
    assert np.linalg.norm(without[-20:] - want[-20:]) > 0.2 * np.linalg.norm(want[-20:])
    cache = types.SimpleNamespace(state=torch.zeros((2, 2 * 16 * 32), dtype=torch.float32, device=DEV))
    got, at = [], 0
    for c in [300, 63, 2] + [1] * 35:
        got.append(_flat(part.forward(h[at: at + c].to(DEV), _ctx([at], [c], [1]), cache)))
        at += c
    got = torch.cat(got)
    assert _rel(got, want) < 2e-5 and _rel(got[-20:], want[-20:]) < 2e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("inner, blocks, taps", [(48, 3, 3), (256, 1, 1), (30, 5, 4), (8, 1, 2), (300, 2, 7), (1, 1, 1), (1100, 4, 4)])
def test_the_gated_linear_recurrence_alone_whole_and_in_portions(inner, blocks, taps, dtype):
    """Portions shorter than the convolution's taps, entries of hundreds of tokens (walked in stretches side by side)
    beside single tokens, against the plain recurrence from a zero state."""
    from atoma_infer_amd.parts import GatedLinearRecurrence
    width = 64
    part = GatedLinearRecurrence(width, inner, blocks, taps)
    w = _drawn(part, "r.", 5, boost=(("y", 6), ("x", 6), ("ra", 2), ("ri", 2)))
    w["lam"] = (w["lam"] - 1.0).to(torch.bfloat16).float()
    _load(part, w, dtype)
    hs = _inputs((467, 129), width, inner)
    m = {"width": inner, "conv": taps, "blocks": blocks}
    want = [pb.gated_linear_recurrence(h.double().numpy(), as_numpy(w, "m."), "m.", m)[0] for h in hs]
    got = _recurrent_case(part, hs, dtype, taps * inner)
    for r in range(2):
        # (float32: the gates' products, the convolution and hundreds of steps of the recurrence each round)
        assert _rel(got[r], want[r]) < (5e-5 if dtype is torch.float32 else PART_TOL[dtype]), r


def test_two_normed_branches_are_averaged_with_their_biases():
    from atoma_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(3)
    t, width = 9, 200
    a, b = torch.randn(3, t, width, generator=g), torch.randn(t, width, generator=g).to(torch.bfloat16)
    wa, wb, ba = torch.randn(width, generator=g), torch.randn(width, generator=g), torch.randn(width, generator=g)
    want = 0.5 * (pb.unit_rms((a.double().sum(0) + ba.double()).numpy(), 1e-5) * wa.double().numpy()
                  + pb.unit_rms(b.double().numpy(), 1e-5) * wb.double().numpy())
    got = ops.normed_branches(a.to(DEV), b.to(DEV), wa.to(DEV), wb.to(DEV), 1e-5, 0.5, ba.to(DEV), None)
    assert _rel(got.cpu(), want) < 1e-6


# ---- the attentions alone -------------------------------------------------------------------------------------------

def _paged_case(part, plain, dtype, lens_and_cuts, page, seed, width=64, hs=None):
    """A mixer over a paged cache on hand-made steps over pages that are dealt out of order: per request the outputs
    of all its portions, and the plain function's on the whole request."""
    lens = [sum(c for r2, c in sum(lens_and_cuts, []) if r2 == r) for r in range(2)]
    g = torch.Generator().manual_seed(seed)
    hs = hs if hs is not None else [torch.randn(c, width, generator=g).to(torch.bfloat16).float() for c in lens]
    want = [plain(h.double().numpy()) for h in hs if len(h)]
    cs = part.cache_spec()
    n_pages = sum(-(-c // page) for c in lens) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    tables = [[order.pop() for _ in range(-(-c // page))] for c in lens]
    max_blocks = max(len(tb) for tb in tables)
    k = torch.zeros((n_pages, cs.kv_heads, page * cs.head_size), dtype=dtype, device=DEV)
    v = torch.zeros_like(k)
    got, at = [[], []], [0, 0]
    for cuts in lens_and_cuts:
        ctx = _ctx([at[r] for r, _ in cuts], [c for _, c in cuts], [0] * len(cuts))
        bt = torch.tensor([tables[r] + [0] * (max_blocks - len(tables[r])) for r, _ in cuts], dtype=torch.int32, device=DEV)
        slots = [tables[r][(at[r] + j) // page] * page + (at[r] + j) % page for r, c in cuts for j in range(c)]
        x = torch.cat([hs[r][at[r]: at[r] + c] for r, c in cuts]).to(DEV, dtype)
        cache = types.SimpleNamespace(k=k, v=v, page_size=page, writable=True, block_tables=bt,
                                      slot_mapping=torch.tensor(slots, dtype=torch.int32, device=DEV))
        y = _flat(part.forward(x, ctx, cache))
        if getattr(part, "out_bias", None) is not None:
            y = y + part.out_bias.cpu()
        o = 0
        for r, c in cuts:
            got[r].append(y[o: o + c])
            o += c
            at[r] += c
    return [torch.cat(x) for x in got if x], want


CUTS = [[(0, 20), (1, 3)], [(0, 1), (1, 1)], [(0, 2)], [(1, 40), (0, 1)], [(0, 50)], [(0, 1)], [(1, 1)], [(0, 1), (1, 2)]]
BOOST = (("q", 30), ("k", 30), ("uq", 3), ("uk", 3), ("dq", 10), ("dkv", 10), ("o", 5), ("g", 10))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m, page", [(latent(16, 4, 40, 24, 8, 24, 0.2), 16), (latent(32, 2, 64, 48, 32, 16, 0.15, 500.0, 16), 32),
                                     (latent(10, 3, 20, 12, 6, 6, 0.4, rot_dims=0), 16), (latent(8, 1, 16, 8, 2, 8, 1.0, 2.0), 48),
                                     (latent(24, 5, 100, 72, 12, 40, 0.1), 16)])
def test_latent_attention_with_a_rotated_key_part_alone(m, page, dtype):
    from atoma_infer_amd.parts import RotaryLatentAttention
    rot = m.get("rot", {"base": 10000.0, "dims": 0})
    part = RotaryLatentAttention(64, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"], m["scale"],
                                 1e-5, rot["base"], rot["dims"])
    w = _drawn(part, "a.", 11, boost=BOOST)
    _load(part, w, dtype)
    plain = lambda h: pb.latent_attention(h, np.arange(len(h)), as_numpy(w, "m."), "m.", m, 1e-5)
    got, want = _paged_case(part, plain, dtype, CUTS, page, m["dim"])
    for g, wt in zip(got, want):
        assert _rel(g, wt) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m, page", [(parallel(32, 4, 2, 0.2, 7, 16, 100.0, (4.0, 64, 8.0, 1.0))["left"], 16),
                                     (parallel(64, 8, 4, 0.125, 33, 64, 500.0)["left"], 32),
                                     (parallel(20, 3, 3, 0.3, 11, 10, 30.0, (2.0, 16, 4.0, 2.0))["left"], 16),
                                     (parallel(16, 1, 1, 0.25, None, 0)["left"], 16),
                                     (parallel(48, 6, 1, 0.1, 64, 24, 1000.0, (8.0, 32, 16.0, 0.5))["left"], 16)])
def test_attention_with_tied_values_biases_chunks_and_a_sink_alone(m, page, dtype):
    from atoma_infer_amd.parts import GatedTiedValueAttention
    rot = m.get("rot", {"base": 10000.0, "dims": 0})
    part = GatedTiedValueAttention(64, m["heads"], m["kv_heads"], m["dim"], m["scale"], rot["base"], rot["dims"],
                                   rot.get("scaling"), chunk=m["mask"]["size"] if "mask" in m else None)
    w = _drawn(part, "t.", 13, boost=BOOST + (("q.b", 20), ("k.b", 20), ("o.b", 5)))
    _load(part, w, dtype)
    plain = lambda h: pb.tied_value_attention(h, np.arange(len(h)), as_numpy(w, "m."), "m.", m)
    got, want = _paged_case(part, plain, dtype, CUTS, page, m["dim"])
    for g, wt in zip(got, want):
        assert _rel(g, wt) < PART_TOL[dtype]


def _marked_inputs(lens, width, mark, size):
    """Column 0 is a mark that one position of one request carries, column 1 is one everywhere."""
    hs = _inputs(lens, width, 3)
    for h in hs:
        h[:, 0], h[:, 1] = 0.0, 1.0
    hs[mark[0]][mark[1], 0] = size
    return hs


@pytest.mark.parametrize("far, chunk", [(3, 64), (63, 64), (64, 64), (0, 150), (149, 150), (130, None)])
def test_one_key_that_stands_out_is_seen_inside_its_chunk_and_not_from_outside(far, chunk):
    """The last column of every key head reads the mark and that of every query head the constant, so the marked
    position scores far above the rest under every later query of its chunk: their outputs are its value.  Queries
    behind the chunk's end do not see it.  In a prompt cut anywhere, and token by token."""
    from atoma_infer_amd.parts import GatedTiedValueAttention
    m = parallel(32, 4, 2, 0.25, chunk, 16, 100.0)["left"]
    part = GatedTiedValueAttention(64, 4, 2, 32, 0.25, 100.0, 16, None, chunk=chunk)
    w = _drawn(part, "k.", 17, boost=(("o", 5),))
    for name, heads, col in (("q", 4, 1), ("k", 2, 0)):
        for a in range(heads):
            w[name][a * 32 + 31] = 0.0
            w[name][a * 32 + 31, col] = 6.0
        w[name + ".b"] = torch.zeros_like(w[name + ".b"])
    _load(part, w, torch.float32)
    total = 260
    hs = _marked_inputs((total, 0), 64, (0, far), 4.0)
    plain = lambda h: pb.tied_value_attention(h, np.arange(len(h)), as_numpy(w, "m."), "m.", m)
    for cuts in ([[(0, 7)], [(0, 121)], [(0, 2)], [(0, 70)], [(0, 60)]], [[(0, 230)]] + [[(0, 1)]] * 30):
        got, want = _paged_case(part, plain, torch.float32, cuts, 16, 1, hs=hs)
        assert _rel(got[0], want[0]) < 2e-5
    # the plain outputs themselves: rows that see the mark differ from a run without it, rows outside do not
    hs0 = [h.clone() for h in hs]
    hs0[0][far, 0] = 0.0
    a, b = plain(hs[0].double().numpy()), plain(hs0[0].double().numpy())
    end = total if chunk is None else min(total, (far // chunk + 1) * chunk)
    moved = np.abs(a - b).max(axis=1) > 1e-3 * np.abs(a).max()
    assert moved[far + 1: end].all() and not moved[end:].any() and not moved[:far].any()


def test_the_sink_takes_its_share_when_no_key_scores():
    """Scores far below zero: the weights of all keys together are small against the sink's one, and the output nearly
    vanishes; without the sink it would be an average of the values."""
    from atoma_infer_amd.parts import GatedTiedValueAttention
    m = parallel(32, 2, 1, 0.5, None, 0)["left"]
    part = GatedTiedValueAttention(64, 2, 1, 32, 0.5, 100.0, 0, None)
    w = _drawn(part, "s.", 19, boost=(("o", 5), ("k", 10)))
    for name, heads, sign in (("q", 2, -1.0), ("k", 1, 1.0)):
        w[name + ".b"] = torch.zeros_like(w[name + ".b"])
        for a in range(heads):
            w[name + ".b"][a * 32 + 31] = 5.0 * sign          # every score gets -25 * scale from this column
            w[name][a * 32 + 31] = 0.0
    _load(part, w, torch.float32)
    plain = lambda h: pb.tied_value_attention(h, np.arange(len(h)), as_numpy(w, "m."), "m.", m)
    got, want = _paged_case(part, plain, torch.float32, [[(0, 40)], [(0, 1)], [(0, 1)]], 16, 5)
    assert _rel(got[0], want[0]) < 2e-5
    m2 = dict(m)
    h = _inputs([42], 64, 5)[0].double().numpy()
    no_bias = {k: v for k, v in as_numpy(w, "m.").items()}
    with_sink = np.linalg.norm(plain(h) - no_bias["m.o.b"])
    assert with_sink < 0.05 * np.linalg.norm(no_bias["m.o"]) * 1.0 + 1e-9 or with_sink < 1.0


def test_a_far_latent_among_hundreds_is_found_by_the_query_that_asks_for_it():
    """The latent's first column carries a mark through W_dkv, and every head's key and query read it: position 5's
    key stands out for all later queries, hundreds of tokens and many pages away, in a prompt and token by token."""
    from atoma_infer_amd.parts import RotaryLatentAttention
    m = latent(16, 2, 32, 16, 8, 16, 0.5, 100.0)
    part = RotaryLatentAttention(64, 2, 16, 8, 16, 32, 16, 0.5, 1e-5, 100.0, 8)
    w = _drawn(part, "f.", 23, boost=(("o", 5), ("uv", 2)))
    w["dkv"][0] = 0.0
    w["dkv"][0, 0] = 8.0                      # latent column 0 = the mark
    w["dq"][0] = 0.0
    w["dq"][0, 1] = 8.0                       # query latent column 0 = the constant
    for a in range(2):
        w["uk"][a * 16 + 15] = 0.0
        w["uk"][a * 16 + 15, 0] = 4.0
        w["uq"][a * 24 + 15] = 0.0
        w["uq"][a * 24 + 15, 0] = 4.0
    _load(part, w, torch.float32)
    total = 330
    hs = _marked_inputs((total, 0), 64, (0, 5), 6.0)
    plain = lambda h: pb.latent_attention(h, np.arange(len(h)), as_numpy(w, "m."), "m.", m, 1e-5)
    for cuts in ([[(0, 3)], [(0, 300)], [(0, 27)]], [[(0, 290)]] + [[(0, 1)]] * 40):
        got, want = _paged_case(part, plain, torch.float32, cuts, 16, 1, hs=hs)
        assert _rel(got[0], want[0]) < 3e-5 and _rel(got[0][-30:], want[0][-30:]) < 3e-5
    hs0 = [h.clone() for h in hs]
    hs0[0][5, 0] = 0.0
    a, b = plain(hs[0].double().numpy()), plain(hs0[0].double().numpy())
    assert np.linalg.norm(a[-30:] - b[-30:]) > 0.2 * np.linalg.norm(a[-30:])


# ---- the whole model ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_prompts_portions_and_single_tokens_agree_with_the_plain_model(dirs, name, dtype):
    d = dirs[name]
    vocab = plain_config(d)["vocab"]
    toks = tokens(150, vocab, 7)
    want = oracle(d, toks)
    runner = make_runner(d, dtype, 256, 16, 2)
    schedules = {"whole": [[(0, 150)]],
                 "tokens": [[(0, 1)]] * 150,
                 "portions": [[(0, c)] for c in (5, 2, 1, 1, 9, 2, 30, 1, 33, 2, 16, 16, 3, 29)],
                 "prompt then tokens": [[(0, 97)]] + [[(0, 1)]] * 53}
    for what, sched in schedules.items():
        got = run_schedule(runner, {0: toks}, sched)[0]
        assert_logits(got, want, dtype, what)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_batches_of_unequal_requests_equal_each_alone_over_pages_and_slots_used_again(dirs, name, dtype):
    """Five requests through a pool of three slots and just enough pages: portions of some beside single tokens of
    others; a request that ends gives its pages and its slot to the next."""
    d = dirs[name]
    vocab = plain_config(d)["vocab"]
    reqs = {r: tokens(n, vocab, 20 + r) for r, n in enumerate((70, 33, 90, 2, 41))}
    want = {r: oracle(d, t) for r, t in reqs.items()}
    runner = make_runner(d, dtype, 256, 16, 3)
    sched = [[(0, 30), (1, 5)], [(0, 1), (1, 28), (2, 17)], [(0, 39), (2, 1)], [(2, 40), (3, 2)], [(2, 1), (4, 1)],
             [(2, 31), (4, 40)]]
    got = run_schedule(runner, reqs, sched)
    for r in reqs:
        assert_logits(got[r], want[r], dtype, r)


@pytest.mark.parametrize("seed", [3, 14, 27, 40, 58, 81, 96, 111])
def test_configurations_drawn_at_random_agree_with_the_plain_model(tmp_path, seed):
    """Layers of the three kinds in any order with sizes drawn at random, loops anywhere, one to five copies of the
    stream or none: a whole prompt, a prompt and single tokens, portions, and a mixed batch over four slots."""
    import random
    cfg = random_config(random.Random(seed))
    d = write_model(str(tmp_path / "m"), cfg, seed, _lively)
    reqs = {r: tokens(n, cfg["vocab"], 100 * seed + r) for r, n in enumerate((230, 33, 150, 2, 77))}
    want = {r: oracle(d, t) for r, t in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(d, dtype, 512, 16, 4)
        runs = {"whole": run_schedule(runner, {0: reqs[0]}, [[(0, 230)]]),
                "tokens": run_schedule(runner, {0: reqs[0]}, [[(0, 190)]] + [[(0, 1)]] * 40),
                "portions": run_schedule(runner, {0: reqs[0]}, [[(0, c)] for c in (5, 2, 60, 1, 33, 2, 100, 3, 24)]),
                "mixed": run_schedule(runner, reqs, [[(0, 100), (1, 5)], [(0, 1), (1, 28), (2, 17)], [(0, 100), (2, 1), (3, 1)],
                                                     [(0, 29), (2, 40), (3, 1)], [(2, 1), (4, 1)], [(2, 91), (4, 76)]])}
        for what, got in runs.items():
            for r, rows in got.items():
                e = row_errors(rows, want[r])
                if dtype == "float32":
                    assert float(e.max()) < TOL[dtype], (what, r, float(e.max()))
                else:
                    # random weights of some configurations leave rows whose logits hardly differ from each other, where
                    # rounding weighs more: half of the rows within half of the tolerance, nine in ten within it
                    assert float(e.median()) < TOL[dtype] / 2 and float((e < TOL[dtype]).double().mean()) >= 0.9, \
                        (what, r, float(e.median()))


def test_long_decoding_over_many_chunks_and_pages(dirs):
    d = dirs["A"]
    toks = tokens(420, plain_config(d)["vocab"], 9)
    want = oracle(d, toks)
    runner = make_runner(d, "float32", 448, 16, 1)
    got = run_schedule(runner, {0: toks}, [[(0, 20)]] + [[(0, 1)]] * 400)[0]
    assert_logits(got, want, "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine_and_its_scheduler(dirs, dtype):
    """Requests of unequal lengths through ``LlmEngine.generate``: continuous batching with prompts in portions (a token
    budget below the longest prompt) beside decoding requests, greedy tokens against the plain model."""
    from atoma_infer_amd.config.engine import CacheConfig, SchedulerConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling.params import GenerateParameters
    d = dirs["A"]
    cfg, w = plain_config(d), numpy_weights(d)
    prompts = [tokens(n, cfg["vocab"], 60 + n) for n in (3, 41, 17, 1, 29)]
    eng = LlmEngine(d, dtype, cache=CacheConfig(block_size=16, num_gpu_blocks_override=24),
                    scheduler=SchedulerConfig(max_num_batched_tokens=24, max_num_sequences=4, max_model_len=128,
                                              enable_chunked_prefill=True))
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=12, ignore_eos_token=True))
    off = 0
    for p, o in zip(prompts, outs):
        got = o.inference_outputs[0].token_ids
        assert len(got) == 12
        rows = pb.forward(list(p) + got, w, cfg)[0][len(p) - 1: -1]
        for step, tok in enumerate(got):
            gap = float(rows[step].max() - rows[step][tok])
            off += gap > (1e-4 if dtype == "float32" else 0.08) * float(np.abs(rows[step]).max())
    assert off == 0, off


def test_the_trace_program_and_the_command_line_run_the_design(dirs, tmp_path):
    import subprocess
    import sys
    d = dirs["D"]
    toks = tokens(30, plain_config(d)["vocab"], 8)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": toks[:9], "want": [0, 8]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": toks[9:], "want": [20]},
                                     {"id": "y", "tokens": toks[:4], "want": [3]}], "end": ["x", "y"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "out")
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                           "--out", out, "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1"]
    want = oracle(d, toks)
    a = torch.from_numpy(np.fromfile(os.path.join(out, "0.f32"), dtype="<f4").reshape(2, -1))
    b = torch.from_numpy(np.fromfile(os.path.join(out, "1.f32"), dtype="<f4").reshape(2, -1))
    assert float(row_errors(a, want[[0, 8]]).max()) < TOL["float32"]
    assert float(row_errors(b, want[[29, 3]]).max()) < TOL["float32"]


def test_the_command_line_writes_random_weights_and_generates(tmp_path):
    """``random-weights`` from a config.json of the design, then ``generate``: greedy tokens are the plain model's, and
    sampling with a seed (temperature, top-k, top-p through the framework's sampler) gives the same tokens twice."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=root)
    cfg_file, d = tmp_path / "config.json", str(tmp_path / "m")
    cfg_file.write_text(json.dumps(BAF_A))
    run = lambda *a: subprocess.run([sys.executable, "-m", "atoma_infer_amd", *a], capture_output=True, text=True, env=env,
                                    timeout=300, cwd=root)
    proc = run("random-weights", "--config", str(cfg_file), "--out", d, "--seed", "4", "--norm-jitter", "0.1")
    assert proc.returncode == 0, proc.stderr[-2000:]
    prompt = tokens(9, BAF_A["vocab"], 2)
    common = ["generate", "--model", d, "--block-size", "16", "--num-gpu-blocks-override", "16", "--max-model-len", "64",
              "--max-num-batched-tokens", "64", "--max-num-sequences", "4", "--max-new-tokens", "6", "--ignore-eos-token",
              "--prompt-ids", ",".join(str(t) for t in prompt)]
    proc = run(*common, "--dtype", "f32", "--greedy")
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = json.loads(proc.stdout.strip().splitlines()[-1])["inference_outputs"][0]["token_ids"]
    w, cfg, seq = numpy_weights(d), plain_config(d), list(prompt)
    for _ in range(6):
        seq.append(int(pb.forward(seq, w, cfg)[0][-1].argmax()))
    assert got == seq[len(prompt):]
    drawn = []
    for _ in range(2):
        proc = run(*common, "--dtype", "bf16", "--temperature", "1.5", "--top-k", "20", "--top-p", "0.9", "--random-seed", "11")
        assert proc.returncode == 0, proc.stderr[-2000:]
        drawn.append(json.loads(proc.stdout.strip().splitlines()[-1])["inference_outputs"][0]["token_ids"])
    assert drawn[0] == drawn[1] and len(drawn[0]) == 6 and all(0 <= t < BAF_A["vocab"] for t in drawn[0])


def test_decode_steps_replayed_as_graphs_equal_the_direct_ones(dirs):
    """Decode steps of one shape are recorded the second time they are seen and replayed afterwards, with the program's
    own direct work between the replays (a prompt of another request): every replay against the plain model."""
    d = dirs["B"]
    vocab = plain_config(d)["vocab"]
    reqs = {0: tokens(60, vocab, 1), 1: tokens(45, vocab, 2), 2: tokens(30, vocab, 3)}
    want = {r: oracle(d, t) for r, t in reqs.items()}
    runner = make_runner(d, "float32", 256, 16, 3)
    assert runner.use_graphs
    sched = [[(0, 20), (1, 5)]] + [[(0, 1), (1, 1)]] * 10 + [[(2, 30)]] + [[(0, 1), (1, 1)]] * 30
    got = run_schedule(runner, reqs, sched)
    for r in (0, 1, 2):
        n = len(got[r])
        assert_logits(got[r], want[r][:n], "float32", r)
