"""Rakuvik on the GPU against the plain implementation: every mechanism alone, then the whole model through the
runner's step function (portions, batches, pages and slots used again) and through the engine's own entry point."""
import copy
import types

import numpy as np
import pytest
import torch

import plain_rakuvik as pr
from rakuvik_util import RAK_A, RAK_B, RAK_C, RAK_D, attention, config, dense, layer, mingru, moe
from somesun_util import logit_err, make_runner, plain_config, plain_weights, row_errors, run_schedule, tokens, write_model

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# float32: the engine's sums run in another order than the plain model's float64 ones; bfloat16: activations are
# rounded to 8 bits about ten times a layer
TOL = {"float32": 3e-5, "bfloat16": 4e-2}
PART_TOL = {torch.float32: 2e-5, torch.bfloat16: 2.5e-2}


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("rakuvik")
    return {n: write_model(str(root / n), c, 31 + i) for i, (n, c) in
            enumerate((("A", RAK_A), ("B", RAK_B), ("C", RAK_C), ("D", RAK_D)))}


def oracle(path, toks):
    return pr.forward(list(toks), plain_weights(path), plain_config(path)).float()


def assert_logits(got, want, dtype, what=""):
    """float32: every row within the tolerance.  bfloat16: rounding moves a router's scores, so now and then a token
    of random weights goes to another expert than in the plain model, and the recurrence carries that on: half of the
    rows within half of the tolerance and nine in ten within it, which no fault of a cache, a state or a mask passes."""
    e = row_errors(got, want)
    if dtype == "float32":
        assert float(e.max()) < TOL[dtype], (what, float(e.max()), int(e.argmax()))
    else:
        assert float(e.median()) < TOL[dtype] / 2 and float((e < TOL[dtype]).double().mean()) >= 0.9, \
            (what, float(e.median()), float((e < TOL[dtype]).double().mean()))


def _ctx(starts, counts, slots):
    """What a mixer reads of a step, for entries of ``counts`` tokens at ``starts``, built by hand."""
    t = int(sum(counts))
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    seq = [e for e, c in enumerate(counts) for _ in range(c)]
    pos = [s + j for s, c in zip(starts, counts) for j in range(c)]
    q_start = np.concatenate([[0], np.cumsum(counts)]).tolist()
    return types.SimpleNamespace(n_tokens=t, n_entries=len(counts), positions=i32(pos), token_seq=i32(seq),
                                 q_start=i32(q_start), state_slots=i32(slots), h_starts=np.asarray(starts, dtype=np.int32),
                                 h_counts=np.asarray(counts, dtype=np.int32), plans={}, scratch={}, decode_bucket=None)


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
    """A sublayer's output as one tensor: planes and weighted terms summed as the norm behind it would."""
    from atoma_infer_amd.parts.base import WeightedSum
    if isinstance(y, WeightedSum):
        return sum(_flat(t) * s for t, s in y.terms)
    return (y.sum(0) if y.dim() == 3 else y).float().cpu()


def _rel(a, b):
    return float((a.double() - b.double()).norm() / b.double().norm())


# ---- small kernels ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("width, n, planes", [(64, 2, (1, 0)), (200, 5, (3, 1)), (4100, 3, (1, 0)), (50, 9, (2, 1)), (33, 2, (1, 1))])
def test_a_layer_s_result_is_kept_and_the_stream_becomes_the_weighted_sum_of_all(width, n, planes):
    """One kernel: X = resid + norm(sum of the sublayer's planes) with one number as the norm's weight, kept as
    results[n - 1]; resid = sum_j w[j] results[j]; and the next norm of that, in either dtype or not at all."""
    from atoma_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(width + n)
    t, eps = 5, 3e-6
    earlier = torch.randn(n - 1, t, width, generator=g)
    resid = torch.randn(t, width, generator=g)
    terms = [(torch.randn(planes[0], t, width, generator=g), 1.0)]
    if planes[1]:
        terms.append((torch.randn(planes[1], t, width, generator=g).to(torch.bfloat16), 1.0))
    g_post, g_next = 0.7, 1.3
    weights = torch.randn(n, generator=g)
    delta = sum(x.double().sum(0) * s for x, s in terms)
    want_x = resid.double() + pr.scalar_norm(delta, torch.tensor(g_post, dtype=torch.float64), eps)
    want_resid = (weights[:-1].double()[:, None, None] * earlier.double()).sum(0) + float(weights[-1]) * want_x
    want_out = pr.scalar_norm(want_resid, torch.tensor(g_next, dtype=torch.float64), 2e-6)
    dev_terms = [((x[0] if x.shape[0] == 1 else x).contiguous().to(DEV), s) for x, s in terms]
    full = lambda v: torch.full((width,), v, dtype=torch.float32, device=DEV)
    for out_dtype in (torch.float32, torch.bfloat16, None):
        results = torch.zeros(n + 2, t, width, device=DEV)
        results[: n - 1] = earlier.to(DEV)
        results[n:] = 5.0                        # rows of later layers: neither read nor written
        r = resid.to(DEV)
        if out_dtype is None:
            out = ops.depth_average(r, dev_terms, full(g_post), eps, results, n, weights.to(DEV))
            assert out is None
        else:
            out = ops.depth_average(r, dev_terms, full(g_post), eps, results, n, weights.to(DEV), full(g_next), 2e-6, out_dtype)
            assert (out.float().cpu().double() - want_out).abs().max() < (3e-5 if out_dtype is torch.float32 else 4e-2)
        assert (results[n - 1].cpu().double() - want_x).abs().max() < 2e-5
        assert (r.cpu().double() - want_resid).abs().max() < 3e-5
        assert bool((results[n:] == 5.0).all()) and torch.equal(results[: n - 1].cpu(), earlier)


@pytest.mark.parametrize("experts, top", [(1, 1), (3, 1), (4, 4), (8, 3), (37, 6), (128, 8)])
def test_softmax_scores_chosen_with_the_correction_and_weighed_without(experts, top):
    from atoma_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(experts)
    z = torch.randn(19, experts, generator=g) * 2
    corr = torch.randn(experts, generator=g) * 0.3
    s = torch.softmax(z.double(), -1)
    want_ids = torch.topk(s + corr.double(), top, dim=-1).indices
    want_w = torch.gather(s, 1, want_ids) * 1.7
    ids, w = ops.route_topk(z.to(DEV), top, "softmax", corr.to(DEV), 1.7)
    order = ids.cpu().long().argsort(-1)
    assert torch.equal(ids.cpu().long().gather(1, order), want_ids.sort(-1).values)
    assert (w.cpu().double().gather(1, order) - want_w.gather(1, want_ids.argsort(-1))).abs().max() < 1e-6
    # the choice is the correction's where it outweighs the scores: it differs from the scores' own order somewhere
    if 1 < top < experts:
        assert not torch.equal(want_ids.sort(-1).values, torch.topk(s, top, dim=-1).indices.sort(-1).values)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, ff", [(64, 48), (40, 20), (128, 96), (200, 1), (384, 768)])
def test_gated_feed_forward_with_the_tanh_form_of_gelu(width, ff, dtype):
    from atoma_infer_amd.parts.base import make_part
    part = make_part("feed_forward", "swiglu", width=width, intermediate=ff, names=("gate", "up", "down"),
                     activation="gelu_tanh")
    w = _drawn(part, "f.", 3, boost=(("gate", 20), ("up", 5)))
    _load(part, w, dtype)
    g = torch.Generator().manual_seed(ff)
    for t in (1, 7, 70):
        h = torch.randn(t, width, generator=g).to(torch.bfloat16).float()
        want = pr.dense_ff(h.double(), {"m." + k: v.double() for k, v in w.items()}, "m.")
        got = _flat(part.forward(h.to(DEV, dtype), None))
        assert _rel(got, want) < PART_TOL[dtype], t


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, mlp", [(64, moe(ff=32, experts=4, top=2, scale=1.5, shared=32)),
                                        (40, moe(ff=24, experts=5, top=5, scale=0.5, shared=8)),
                                        (128, moe(ff=64, experts=8, top=3, scale=2.0, shared=0)),
                                        (64, moe(ff=32, experts=1, top=1, scale=1.0, shared=96)),
                                        (96, moe(ff=40, experts=3, top=1, scale=0.7, shared=20)),
                                        (384, moe(ff=160, experts=32, top=4, scale=1.8, shared=224)),
                                        (320, moe(ff=96, experts=16, top=3, scale=2.5, shared=64))])
def test_routed_experts_alone(width, mlp, dtype):
    """Softmax scores, a correction large enough to change the choice, squared-ReLU experts weighed on their outputs,
    no renormalising (all experts chosen: the weights sum to the scale; one expert: its score is 1), and the expert
    that every token uses behind its gate.  Widths that the matrix-core products take and that they do not."""
    from atoma_infer_amd.parts.base import make_part
    r = mlp["router"]
    part = make_part("feed_forward", "routed_experts", width=width, intermediate=mlp["expert"]["ff"], experts=r["experts"],
                     top=r["top"], score="softmax", scale=r["scale"], correction=True, expert="relu2",
                     shared=mlp["shared"]["ff"] if "shared" in mlp else 0)
    w = _drawn(part, "e.", 7, boost=(("router", 3), ("correction", 2)))
    _load(part, w, dtype)
    pw = {"m." + k: v.double() for k, v in w.items()}
    g = torch.Generator().manual_seed(width)
    for t in (1, 9, 150):
        h = torch.randn(t, width, generator=g).to(torch.bfloat16).float()
        want = pr.moe_ff(h.double(), pw, "m.", mlp)
        got = _flat(part.forward(h.to(DEV, dtype), None))
        if dtype is torch.float32:
            assert _rel(got, want) < PART_TOL[dtype], t
            continue
        # bfloat16: a token whose choice is a close call may go to another expert; every other token is held to
        # the tolerance (the router's logits are float32 sums of bfloat16 products: far more exact than the gap asked)
        e = (got.double() - want).norm(dim=-1) / want.norm(dim=-1).clamp_min(1e-9)
        choice = torch.softmax(h.double() @ pw["m.router"].T, -1) + pw["m.correction"]
        ranked = choice.sort(-1, descending=True).values
        clear = torch.ones(t, dtype=torch.bool) if r["top"] == r["experts"] else \
            (ranked[:, r["top"] - 1] - ranked[:, r["top"]]) > 2e-3
        assert float(clear.double().mean()) > 0.8 and float(e[clear].max()) < 2 * PART_TOL[dtype], (t, float(e[clear].max()))
    if 1 < r["top"] < r["experts"]:
        ids, _ = pr.route(h.double(), pw, "m.", r)
        plain_ids = torch.topk(torch.softmax(h.double() @ pw["m.router"].T, -1), r["top"], dim=-1).indices
        assert not torch.equal(ids.sort(-1).values, plain_ids.sort(-1).values)


# ---- the recurrence alone ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("inner", [1, 40, 256, 300, 1100])
def test_mingru_alone_whole_and_in_portions(inner, dtype):
    """Two requests side by side, cut into portions of one token, two, a few, and of hundreds (those are walked in
    stretches side by side, the short ones token by token, both kinds in one step too), each carried by its state
    slot; against the plain recurrence from a zero state."""
    from atoma_infer_amd.parts import MinGRU
    width = 64
    part = MinGRU(width, inner)
    w = _drawn(part, "x.", 5, boost=(("z", 8), ("x", 12), ("g", 8)))
    _load(part, w, dtype)
    g = torch.Generator().manual_seed(inner)
    lens = (467, 129)
    hs = [torch.randn(c, width, generator=g).to(torch.bfloat16).float() for c in lens]
    pw = {"r." + k: v.double() for k, v in w.items()}
    want = [pr.mingru(h.double(), pw, "r.", {"width": inner}) for h in hs]
    # both branches of the candidate occur
    u = hs[0].double() @ pw["r.x"].T + pw["r.x.b"]
    assert bool((u >= 0).any()) and bool((u < 0).any())
    state = torch.full((4, inner), float("nan"), dtype=torch.float32, device=DEV)
    state[1].fill_(7.0)                       # another request's slot must stay as it is
    state[0].zero_()
    state[3].zero_()
    cache = types.SimpleNamespace(state=state)
    got, at = [[], []], [0, 0]
    for cuts in ([(0, 1), (1, 2)], [(0, 2)], [(1, 1), (0, 1)], [(0, 30), (1, 6)], [(0, 3)], [(0, 64), (1, 17)], [(0, 250)],
                 [(0, 16), (1, 100)], [(1, 3), (0, 100)]):
        ctx = _ctx([at[r] for r, _ in cuts], [c for _, c in cuts], [3 if r == 0 else 0 for r, _ in cuts])
        x = torch.cat([hs[r][at[r]: at[r] + c] for r, c in cuts]).to(DEV, dtype)
        y = _flat(part.forward(x, ctx, cache))
        o = 0
        for r, c in cuts:
            got[r].append(y[o: o + c])
            o += c
            at[r] += c
    assert at == list(lens) and bool((state[1] == 7.0).all()) and bool(state[2].isnan().all())
    for r in range(2):
        assert _rel(torch.cat(got[r]), want[r]) < PART_TOL[dtype], r


def test_a_far_token_stays_in_the_recurrent_state():
    """Update gates close to zero and one early token whose candidate is large: hundreds of tokens later the read-out
    still holds it.  A state that is lost, cleared or carried by the wrong slot changes the late outputs entirely."""
    from atoma_infer_amd.parts import MinGRU
    width, inner = 64, 96
    part = MinGRU(width, inner)
    w = _drawn(part, "y.", 9, boost=(("x", 10), ("g", 8)))
    w["z"] = (w["z"] * 0.1).to(torch.bfloat16).float()
    w["z.b"] = torch.full_like(w["z.b"], -6.0)                 # z about 1/400: the state hardly moves
    _load(part, w, torch.float32)
    g = torch.Generator().manual_seed(1)
    count = 400
    h = torch.randn(count, width, generator=g).to(torch.bfloat16).float() * 0.3
    h[5] = h[5] * 200                                           # the far token
    pw = {"r." + k: v.double() for k, v in w.items()}
    want = pr.mingru(h.double(), pw, "r.", {"width": inner})
    h_without = h.clone()
    h_without[5] = h[5] / 200
    assert (pr.mingru(h_without.double(), pw, "r.", {"width": inner})[-20:] - want[-20:]).norm() > 0.2 * want[-20:].norm()
    state = torch.zeros((2, inner), dtype=torch.float32, device=DEV)
    cache = types.SimpleNamespace(state=state)
    got, at = [], 0
    for c in [300, 63, 2] + [1] * 35:
        got.append(_flat(part.forward(h[at: at + c].to(DEV), _ctx([at], [c], [1]), cache)))
        at += c
    got = torch.cat(got)
    assert _rel(got, want) < 2e-5 and _rel(got[-20:], want[-20:]) < 2e-5


# ---- differential attention alone ------------------------------------------------------------------------------------

def _paged_case(parts, plains, dtype, lens_and_cuts, page, seed, mark=None, width=64):
    """Mixers over one paged cache (the first writes it, the others read it) on hand-made steps over pages that are
    dealt out of order: per part and request the outputs of all its portions, and the plain functions' on the whole
    request."""
    lens = [sum(c for r2, c in sum(lens_and_cuts, []) if r2 == r) for r in range(2)]
    g = torch.Generator().manual_seed(seed)
    hs = [torch.randn(c, width, generator=g).to(torch.bfloat16).float() for c in lens]
    if mark is not None:
        # column 0 is a mark that one position of one request carries, column 1 is one everywhere (see ``_marked``)
        r, p, size = mark
        for h in hs:
            h[:, 0], h[:, 1] = 0.0, 1.0
        hs[r][p, 0] = size
    want = [[plain(h.double()) for h in hs if len(h)] for plain in plains]
    cs = parts[0].cache_spec()
    n_pages = sum(-(-c // page) for c in lens) + 3
    order = torch.randperm(n_pages, generator=g).tolist()
    tables = [[order.pop() for _ in range(-(-c // page))] for c in lens]
    max_blocks = max(len(tb) for tb in tables)
    k = torch.zeros((n_pages, cs.kv_heads, page * cs.head_size), dtype=dtype, device=DEV)
    v = torch.zeros_like(k)
    got, at = [[[], []] for _ in parts], [0, 0]
    for cuts in lens_and_cuts:
        ctx = _ctx([at[r] for r, _ in cuts], [c for _, c in cuts], [0] * len(cuts))
        bt = torch.tensor([tables[r] + [0] * (max_blocks - len(tables[r])) for r, _ in cuts], dtype=torch.int32, device=DEV)
        slots = [tables[r][(at[r] + j) // page] * page + (at[r] + j) % page for r, c in cuts for j in range(c)]
        x = torch.cat([hs[r][at[r]: at[r] + c] for r, c in cuts]).to(DEV, dtype)
        for i, part in enumerate(parts):
            cache = types.SimpleNamespace(k=k, v=v, page_size=page, writable=i == 0, block_tables=bt,
                                          slot_mapping=torch.tensor(slots, dtype=torch.int32, device=DEV))
            y = _flat(part.forward(x, ctx, cache))
            o = 0
            for r, c in cuts:
                got[i][r].append(y[o: o + c])
                o += c
        for r, c in cuts:
            at[r] += c
    return [[torch.cat(x) for x in gp if x] for gp in got], want


CUTS = [[(0, 20), (1, 3)], [(0, 1), (1, 1)], [(0, 2)], [(1, 40), (0, 1)], [(0, 50)], [(0, 1)], [(1, 1)], [(0, 1), (1, 2)]]
BOOST = (("q", 30), ("k", 30), ("v", 10), ("o", 5), ("g", 10))


def _difference_tensors(w, seed):
    """The four small tensors of the difference's weight, large enough that it is far from the configuration's
    constant: a map that is dropped, or swapped with the other, then shows."""
    g = torch.Generator().manual_seed(seed)
    for n, f in (("lq1", 0.5), ("lk1", 0.5), ("lq2", 0.3), ("lk2", 0.3)):
        w[n] = (torch.randn(w[n].shape, generator=g) * f * (8.0 / w[n].numel()) ** 0.5).to(torch.bfloat16).float()
    w["lk1"] = (w["lq1"] * 0.4).to(torch.bfloat16).float()             # exp of a positive sum: above 1
    return w


def _marked(w, m, size):
    """Makes the last column of every map (one that is not rotated) of the keys read input column 0 and that of the
    queries input column 1, ``size`` times: a position whose input column 0 is A, among positions where it is zero,
    scores size^2 A scale above the rest under every query whose input column 1 is one."""
    rows = lambda heads: [a * m["dim"] + m["dim"] - 1 for a in range(2 * heads)]
    for name, heads, col in (("q", m["heads"], 1), ("k", m["kv_heads"], 0)):
        if name in w:
            w[name][rows(heads)] = 0.0
            w[name][rows(heads), col] = size
    return w


def _diff_parts(m, dtype, seed=7, width=64, reader=True, eps=1e-5, boost=None, mark=None):
    """The part that owns the cache and, with ``reader``, one of other weights that reads it."""
    from atoma_infer_amd.parts import DifferentialAttention
    rot = m.get("rot")
    kw = dict(width=width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_size=m["dim"], value_size=m["vdim"],
              scale=m["scale"], diff=m["diff"], norm_eps=eps, rotary_base=rot["base"] if rot else 1.0,
              rotary_dim=rot["dims"] if rot else 0, rotary_factor=(rot.get("scaling") or {}).get("factor", 1.0) if rot else 1.0)
    own = DifferentialAttention(owns_cache=True, **kw)
    boost = BOOST if boost is None else boost
    w = _difference_tensors(_drawn(own, "t.", seed, boost=boost), seed)
    if mark:
        _marked(w, m, mark)
    _load(own, w, dtype)
    pw = {"a." + k: v.double() for k, v in w.items()}
    parts, plains = [own], [lambda h: pr.differential_attention(h, pw, "a.", m, eps)]
    assert abs(pr.difference_weight(pw, "a.", m) - m["diff"]) > 0.05
    if reader:
        other = DifferentialAttention(owns_cache=False, **kw)
        assert "k" not in other.weight_specs() and "v" not in other.weight_specs()
        w2 = _difference_tensors(_drawn(other, "u.", seed + 1, boost=boost), seed + 1)
        if mark:
            _marked(w2, m, mark)
        _load(other, w2, dtype)
        pw2 = {"b." + k: v.double() for k, v in w2.items()}
        parts.append(other)
        plains.append(lambda h: pr.differential_attention(h, pw2, "b.", m, eps, kv=pr.keys_and_values(h, pw, "a.", m)))
    return parts, plains


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m, page", [
    (attention(dim=16, heads=4, kv_heads=2, vdim=24, scale=0.3, diff=0.2, rot_dims=8, base=100.0, factor=4.0), 16),
    (attention(dim=32, heads=4, kv_heads=4, vdim=64, scale=0.18, diff=0.4, rot_dims=32, base=500.0), 16),
    (attention(dim=64, heads=2, kv_heads=1, vdim=32, scale=0.12, diff=0.1, rot_dims=None), 32),
    (attention(dim=6, heads=1, kv_heads=1, vdim=5, scale=1.0, diff=0.5, rot_dims=2, base=2.0, factor=1.0), 16),
    (attention(dim=20, heads=6, kv_heads=3, vdim=48, scale=0.2, diff=0.3, rot_dims=20, base=30.0, factor=8.0), 4),
    (attention(dim=8, heads=2, kv_heads=1, vdim=40, scale=0.4, diff=0.6, rot_dims=4, base=10.0), 16),
    (attention(dim=64, heads=8, kv_heads=2, vdim=128, scale=0.1, diff=0.35, rot_dims=64, base=1e4, factor=2.0), 16),
    (attention(dim=40, heads=3, kv_heads=3, vdim=72, scale=0.15, diff=0.25, rot_dims=40, base=300.0, factor=2.5), 16),
    (attention(dim=48, heads=5, kv_heads=1, vdim=64, scale=0.14, diff=0.7, rot_dims=16, base=1e5), 16),
    (attention(dim=72, heads=2, kv_heads=2, vdim=160, scale=0.1, diff=0.45, rot_dims=36, base=50.0, factor=16.0), 16),
    (attention(dim=128, heads=2, kv_heads=1, vdim=200, scale=0.09, diff=0.15, rot_dims=128, base=1e4), 16),
])
def test_differential_attention_alone_and_a_layer_that_reads_its_cache(m, page, dtype):
    """Values narrower than both maps together, as wide, and wider; part of a map rotated, all of it, none; the
    rotation slowed or not; one head and grouped heads (two to ten query maps a key head); cached heads of 16 to 256
    columns; pages of 4, 16 and 32 tokens; and beside the part that writes the cache one with queries, gates and a
    difference weight of its own that only reads it."""
    parts, plains = _diff_parts(m, dtype)
    assert parts[0].cache_spec().head_size == -(-max(2 * m["dim"], m["vdim"]) // 16) * 16
    got, want = _paged_case(parts, plains, dtype, CUTS, page, seed=m["dim"])
    # (bfloat16: the two maps' outputs are rounded before a1 - lam a2, which is smaller than either, is normed)
    tol = {torch.float32: 2e-5, torch.bfloat16: 4e-2}[dtype]
    for gp, wp in zip(got, want):
        for a, b in zip(gp, wp):
            assert _rel(a, b) < tol
            assert _rel(a[:3], b[:3]) < tol              # the first tokens of a sequence
    assert _rel(want[0][0], want[1][0]) > 0.3                        # (the reader's rows are not the writer's)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_rotation_tells_positions_apart_far_from_the_start(dtype):
    """Requests that begin with the same tokens but whose portions start at other positions, far enough that an angle
    taken in reduced precision, or a scaling factor that is left out, would show."""
    m = attention(dim=32, heads=2, kv_heads=1, vdim=32, scale=0.3, diff=0.3, rot_dims=32, base=50.0, factor=3.0)
    parts, plains = _diff_parts(m, dtype, reader=False)
    cuts = [[(0, 700), (1, 2)], [(0, 2)], [(0, 1), (1, 1)], [(0, 60)], [(0, 1)], [(0, 1)]]
    got, want = _paged_case(parts, plains, dtype, cuts, 16, seed=2)
    # (a float32 angle at position 700 is exact to about 5e-5, and so are the rows made of it; an angle of fewer
    # bits is off by radians there)
    far = {torch.float32: 1e-4, torch.bfloat16: PART_TOL[dtype]}[dtype]
    assert _rel(got[0][0], want[0][0]) < far and _rel(got[0][0][-64:], want[0][0][-64:]) < far
    # the plain rows change when the factor is left out
    m1 = copy.deepcopy(m)
    m1["rot"]["scaling"]["factor"] = 1.0
    parts1, plains1 = _diff_parts(m1, dtype, reader=False)
    g = torch.Generator().manual_seed(2)
    h = torch.randn(80, 64, generator=g).to(torch.bfloat16).double()
    assert _rel(plains1[0](h), plains[0](h)) > 0.1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_at_a_page_s_last_slot(dtype):
    """One early key, at a page's last slot, that outweighs the hundreds behind it in both maps: every later row, in
    long portions, in portions of two tokens and decoded alone, is made of that key's value, for the layer that owns
    the cache and for the one that reads it.  Without the mark the late rows are other rows altogether."""
    m = attention(dim=32, heads=4, kv_heads=2, vdim=48, scale=0.5, diff=0.3, rot_dims=8, base=200.0)
    small = (("q", 3), ("k", 3), ("v", 10), ("o", 5), ("g", 10))
    parts, plains = _diff_parts(m, dtype, boost=small, mark=4.0)
    cuts = [[(0, 100), (1, 7)], [(0, 500)], [(0, 2), (1, 1)], [(0, 38)]] + [[(0, 1)]] * 12 + [[(0, 2)]] * 3
    got, want = _paged_case(parts, plains, dtype, cuts, 16, seed=5, mark=(0, 15, 4.0))       # 16 x 4 x 0.5 = 32 above
    unmarked = _paged_case(parts, plains, dtype, cuts, 16, seed=5, mark=(0, 15, 0.0))[1]
    for i in range(2):
        assert _rel(got[i][0], want[i][0]) < PART_TOL[dtype] and _rel(got[i][0][-18:], want[i][0][-18:]) < PART_TOL[dtype]
        assert _rel(got[i][1], want[i][1]) < PART_TOL[dtype]
        assert _rel(unmarked[i][0][-18:], want[i][0][-18:]) > 0.3
        assert _rel(unmarked[i][0][:15], want[i][0][:15]) < 1e-9          # the rows before it know nothing of it


# ---- the whole model through the step function --------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_prompts_token_by_token_decoding_and_portions(dirs, name, dtype):
    d = dirs[name]
    vocab = plain_config(d)["vocab"]
    toks = tokens(150, vocab, 3)
    want = oracle(d, toks)
    runner = make_runner(d, dtype, 256, 16, 4)
    n = len(toks)
    schedules = {
        "whole": [[(0, n)]],
        "tokens": [[(0, 1)]] * n,                                        # crosses every page edge one token at a time
        "portions": [[(0, c)] for c in (2, 2, 3, 1, 16, 2, 31, 33, 2, 7, 1, 1, 2, 40, 7)],
        "long decoding": [[(0, 10)]] + [[(0, 1)]] * (n - 10),
        "stretches then tokens": [[(0, 70)], [(0, 2)], [(0, 68)]] + [[(0, 1)]] * 10,
    }
    assert sum(c for s in schedules["portions"] for _, c in s) == n
    for what, sched in schedules.items():
        got = run_schedule(runner, {0: toks}, sched)[0]
        assert_logits(got, want, dtype, what)
    runner.manager.check()
    assert runner.manager.num_requests() == 0


def test_every_layer_s_result_against_the_plain_model(dirs):
    """The stream behind every layer in float32: the weighted sum of the embedding's rows and all results so far."""
    from atoma_infer_amd.engine.step import StepEntry
    for name in ("A", "B"):
        d = dirs[name]
        cfg, w = plain_config(d), plain_weights(d)
        toks = tokens(40, cfg["vocab"], 9)
        streams = [w["embed"][torch.tensor(toks)]]
        pr.forward(toks, w, cfg, streams=streams)
        runner = make_runner(d, "float32", 128, 16, 2)
        seen = {}
        runner.model.after_block = lambda pos, resid, pending: seen.__setitem__(pos, resid.detach().float().cpu().clone())
        runner.add_request(0)
        runner.step([StepEntry(0, toks, 0, [39])])
        assert len(seen) == len(cfg["layers"])
        for i in range(len(cfg["layers"])):
            want = sum(w[f"l{i}.dwa"][j] * streams[j] for j in range(i + 2))
            assert _rel(seen[i], want) < 2e-5, (name, i)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_batches_of_unequal_requests_with_pages_and_slots_used_again(dirs, name, dtype):
    """Up to four live requests, portions beside single tokens, in a pool that holds them only because finished requests
    give their pages and state slots back: every request's logits are those of the request alone."""
    d = dirs[name]
    vocab = plain_config(d)["vocab"]
    reqs = {i: tokens(n, vocab, 20 + i) for i, n in enumerate((70, 1, 45, 130, 2, 64, 33))}
    want = {i: oracle(d, t) for i, t in reqs.items()}
    sched = [[(0, 30), (1, 1)], [(0, 1), (2, 2), (3, 64)], [(0, 1), (2, 1), (3, 2), (4, 1)], [(0, 38), (2, 42), (4, 1)],
             [(3, 1), (5, 17)], [(3, 33), (5, 1), (6, 2)], [(5, 46), (6, 1), (3, 1)], [(6, 30), (3, 29)]]
    runner = make_runner(d, dtype, 320, 16, 4)      # 345 tokens in all: only with pages used again
    got = run_schedule(runner, reqs, sched)
    if dtype == "float32":
        for i in reqs:
            assert_logits(got[i], want[i], dtype, i)
    # bfloat16: all requests' rows together (a request of one or two tokens has too few rows for shares of rows; and
    # behind a recurrence of ONE channel the mixer's normed output is a fixed row times the sign of the token's gate,
    # which rounding turns over where the gate is next to zero: one such token moves its request's next rows)
    e = torch.cat([row_errors(got[i], want[i]) for i in reqs])
    assert float(e.median()) < TOL[dtype] / 2 and float((e < TOL[dtype]).double().mean()) >= 0.9
    runner.manager.check()
    assert runner.manager.num_requests() == 0 and runner.manager.num_free_slots() == 4


def test_decode_steps_replayed_as_graphs_give_the_eager_logits(dirs):
    """Steps in which every entry brings one token are recorded into graphs from their second sighting on; the
    recurrent state and the kept results are read from the step's device tensors."""
    sched = [[(0, 20), (1, 5), (2, 9)]] + [[(0, 1), (1, 1), (2, 1)]] * 40 + [[(1, 15)], [(2, 11)]]
    for name in ("B", "A"):
        d = dirs[name]
        vocab = plain_config(d)["vocab"]
        reqs = {i: tokens(60, vocab, 40 + i) for i in range(3)}
        want = {i: oracle(d, t) for i, t in reqs.items()}
        runner = make_runner(d, "bfloat16", 256, 16, 4)
        assert runner.use_graphs
        got = run_schedule(runner, reqs, sched)
        assert any(g.graph is not None for g in runner._graphs.values())
        for i in reqs:
            assert_logits(got[i], want[i], "bfloat16", (name, i))
        eager = make_runner(d, "bfloat16", 256, 16, 4)
        eager.use_graphs = False
        plain_steps = run_schedule(eager, reqs, sched)
        for i in reqs:
            assert logit_err(got[i], plain_steps[i]) < 1e-3, (name, i)


def test_a_layer_order_of_its_own_and_pages_of_other_sizes(tmp_path):
    """Three attention layers in a row of which the last two read the first one's cache, the recurrence last and
    twice, widths that are no multiple of 32, pages of 32 and 48 tokens."""
    att = dict(dim=12, heads=3, kv_heads=1, vdim=20, scale=0.25, diff=0.15, rot_dims=6, base=10.0, factor=1.5)
    cfg = config([layer("attention", attention(**att), dense(24)),
                  layer("attention", attention(kv_from=0, **att), None),
                  layer("attention", attention(kv_from=0, **att), moe(ff=16, experts=2, top=2, scale=1.0, shared=0)),
                  layer("mingru", mingru(24), None),
                  layer("mingru", mingru(56), dense(20))], width=40, vocab=60, eps=1e-6)
    d = write_model(str(tmp_path / "m"), cfg, 5)
    toks = tokens(70, 60, 1)
    want = oracle(d, toks)
    for dtype, page in (("float32", 32), ("bfloat16", 48), ("bfloat16", 32)):
        runner = make_runner(d, dtype, 192, page, 2)
        got = run_schedule(runner, {0: toks}, [[(0, 3)], [(0, 30)], [(0, 1)], [(0, 2)], [(0, 33)], [(0, 1)]])[0]
        assert_logits(got, want, dtype, (dtype, page))


# ---- through the engine ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine_and_its_scheduler(dirs, dtype):
    """Requests of unequal lengths through ``LlmEngine.generate``: continuous batching with prompts in portions (a token
    budget below the longest prompt) beside decoding requests, greedy tokens against the plain model."""
    from atoma_infer_amd.config.engine import CacheConfig, SchedulerConfig
    from atoma_infer_amd.engine.engine import LlmEngine
    from atoma_infer_amd.sampling.params import GenerateParameters
    d = dirs["A"]
    cfg, w = plain_config(d), plain_weights(d)
    prompts = [tokens(n, cfg["vocab"], 60 + n) for n in (3, 41, 17, 1, 29)]
    eng = LlmEngine(d, dtype, cache=CacheConfig(block_size=16, num_gpu_blocks_override=24),
                    scheduler=SchedulerConfig(max_num_batched_tokens=24, max_num_sequences=4, max_model_len=128,
                                              enable_chunked_prefill=True))
    outs = eng.generate(prompts, GenerateParameters(do_sample=False, max_new_tokens=12, ignore_eos_token=True))
    off = 0
    for p, o in zip(prompts, outs):
        got = o.inference_outputs[0].token_ids
        assert len(got) == 12
        rows = pr.forward(list(p) + got, w, cfg)[len(p) - 1: -1]
        for step, tok in enumerate(got):
            # the engine's token is the plain model's argmax, up to logits that rounding cannot tell apart
            gap = float(rows[step].max() - rows[step][tok])
            off += gap > (1e-4 if dtype == "float32" else 0.08) * float(rows[step].abs().max())
    assert off == 0, off


def test_the_trace_program_runs_the_design(dirs, tmp_path):
    import json
    import os
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
    assert logit_err(a, want[[0, 8]]) < TOL["float32"] and logit_err(b, want[[29, 3]]) < TOL["float32"]


def test_the_command_line_writes_random_weights_and_generates(tmp_path):
    """``random-weights`` from a config.json of the design, then ``generate``: greedy tokens are the plain model's, and
    sampling with a seed (temperature, top-k, top-p through the framework's sampler) gives the same tokens twice."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=root)
    cfg_file, d = tmp_path / "config.json", str(tmp_path / "m")
    cfg_file.write_text(json.dumps(RAK_A))
    run = lambda *a: subprocess.run([sys.executable, "-m", "atoma_infer_amd", *a], capture_output=True, text=True, env=env,
                                    timeout=300, cwd=root)
    proc = run("random-weights", "--config", str(cfg_file), "--out", d, "--seed", "4", "--norm-jitter", "0.1")
    assert proc.returncode == 0, proc.stderr[-2000:]
    prompt = tokens(9, RAK_A["vocab"], 2)
    common = ["generate", "--model", d, "--block-size", "16", "--num-gpu-blocks-override", "16", "--max-model-len", "64",
              "--max-num-batched-tokens", "64", "--max-num-sequences", "4", "--max-new-tokens", "6", "--ignore-eos-token",
              "--prompt-ids", ",".join(str(t) for t in prompt)]
    proc = run(*common, "--dtype", "f32", "--greedy")
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = json.loads(proc.stdout.strip().splitlines()[-1])["inference_outputs"][0]["token_ids"]
    assert got == pr.greedy_generate(prompt, 6, plain_weights(d), plain_config(d))
    drawn = []
    for _ in range(2):
        proc = run(*common, "--dtype", "bf16", "--temperature", "1.5", "--top-k", "20", "--top-p", "0.9", "--random-seed", "11")
        assert proc.returncode == 0, proc.stderr[-2000:]
        drawn.append(json.loads(proc.stdout.strip().splitlines()[-1])["inference_outputs"][0]["token_ids"])
    assert drawn[0] == drawn[1] and len(drawn[0]) == 6 and all(0 <= t < RAK_A["vocab"] for t in drawn[0])


@pytest.mark.parametrize("kind", ["recurrences only", "attention only", "one recurrence"])
def test_models_without_a_cache_or_without_a_state(tmp_path, kind):
    """A model whose layers are all recurrences keeps no pages, one whose layers are all attention no state rows."""
    att = dict(dim=16, heads=2, kv_heads=1, vdim=24, scale=0.25, diff=0.3, rot_dims=8, base=50.0, factor=2.0)
    layers = {"recurrences only": [layer("mingru", mingru(48), dense(40)), layer("mingru", mingru(80), None),
                                   layer("mingru", mingru(24), moe(ff=32, experts=4, top=2, scale=1.2, shared=16))],
              "attention only": [layer("attention", attention(**att), moe(ff=32, experts=3, top=2, scale=0.9, shared=0)),
                                 layer("attention", attention(kv_from=0, **att), dense(48)),
                                 layer("attention", attention(**att), None)],
              "one recurrence": [layer("mingru", mingru(32), None)]}[kind]
    d = write_model(str(tmp_path / "m"), config(layers, width=64, vocab=80), 3)
    reqs = {i: tokens(n, 80, 7 + i) for i, n in enumerate((90, 37, 2))}
    want = {i: oracle(d, t) for i, t in reqs.items()}
    sched = [[(0, 70), (1, 2)], [(0, 1), (1, 1), (2, 2)], [(0, 2), (1, 34)], [(0, 17)]]
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(d, dtype, 192, 16, 4)
        got = run_schedule(runner, reqs, sched)
        e = torch.cat([row_errors(got[i], want[i]) for i in reqs])
        assert float(e.max()) < TOL[dtype] if dtype == "float32" else \
            float(e.median()) < TOL[dtype] / 2 and float((e < TOL[dtype]).double().mean()) >= 0.9, (dtype, float(e.max()))
        runner.manager.check()
        assert runner.manager.num_requests() == 0
