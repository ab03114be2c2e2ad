"""What pins the plain Bafilorn (closed forms worked by hand) and what the configuration and the builder do, on the CPU."""
import copy
import math

import numpy as np
import pytest

import plain_bafilorn as pb
from bafilorn_util import BAF_A, BAF_B, BAF_C, BAF_D, config, latent, layer, lightning, parallel


# ---- the plain implementation ------------------------------------------------------------------------------------

def test_the_pair_table_is_indexed_by_both_tokens_and_the_first_token_takes_the_last_row():
    cfg = {"embedding": {"scale": 2.0, "bigram": {"buckets": 5, "mul_prev": 3, "mul_cur": 2}}}
    w = {"embed": np.arange(12.0).reshape(6, 2), "bigram": 100.0 + np.arange(12.0).reshape(6, 2)}
    x = pb.embed(np.array([4, 1, 5]), w, cfg)
    assert np.allclose(x[0], 2 * w["embed"][4] + w["bigram"][5])                 # row number 'buckets'
    assert np.allclose(x[1], 2 * w["embed"][1] + w["bigram"][(4 * 3 + 1 * 2) % 5])
    assert np.allclose(x[2], 2 * w["embed"][5] + w["bigram"][(1 * 3 + 5 * 2) % 5])
    del cfg["embedding"]["bigram"]
    assert np.allclose(pb.embed(np.array([4]), w, cfg), 2 * w["embed"][[4]])


def test_rotation_pairs_neighbours_or_halves_and_turns_by_the_position():
    x = np.zeros((1, 1, 6))
    x[0, 0] = [1, 0, 0, 0, 0, 7]
    f = np.array([0.5, 0.25])
    a = pb.rotate(x, [2], f, 4, "interleaved")[0, 0]
    assert np.allclose(a, [math.cos(1.0), math.sin(1.0), 0, 0, 0, 7])            # (0, 1) a pair; columns 4, 5 pass
    b = pb.rotate(x, [2], f, 4, "half")[0, 0]
    assert np.allclose(b, [math.cos(1.0), 0, math.sin(1.0), 0, 0, 7])            # (0, 2) a pair
    # scores depend on the distance alone
    g = np.random.default_rng(0)
    q, k = g.standard_normal((1, 1, 6)), g.standard_normal((1, 1, 6))
    for lay in ("interleaved", "half"):
        s1 = (pb.rotate(q, [9], f, 4, lay) * pb.rotate(k, [4], f, 4, lay)).sum()
        s2 = (pb.rotate(q, [105], f, 4, lay) * pb.rotate(k, [100], f, 4, lay)).sum()
        assert abs(s1 - s2) < 1e-9


def test_long_waves_are_slowed_down_short_ones_kept_and_the_band_between_blended():
    base, dims = 10.0, 8
    sc = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    f, mag = pb.yarn_frequencies(base, dims, sc)
    plain = np.array([1.0, 10 ** -0.25, 10 ** -0.5, 10 ** -0.75])
    where = lambda t: dims * math.log(64 / (2 * math.pi * t)) / (2 * math.log(base))
    lo, hi = max(math.floor(where(8.0)), 0), min(math.ceil(where(1.0)), dims - 1)
    assert (lo, hi) == (0, 5)
    ramp = np.clip((np.arange(4) - lo) / (hi - lo), 0, 1)
    assert np.allclose(ramp, [0, 0.2, 0.4, 0.6])
    assert np.allclose(f, plain / 4 * ramp + plain * (1 - ramp))
    assert f[0] == 1.0 and abs(f[3] - plain[3] * (0.6 / 4 + 0.4)) < 1e-12
    assert abs(mag - (0.1 * math.log(4.0) + 1)) < 1e-12
    assert pb.yarn_frequencies(base, dims, None)[1] == 1.0


def test_chunks_sinks_and_groups_of_the_softmax():
    T, d = 6, 2
    q = np.zeros((T, 2, d))
    k = np.zeros((T, 1, d))
    v = np.arange(T, dtype=float).reshape(T, 1, 1) + 1
    # all scores zero: position i averages the values it sees; with a sink the denominator has one term more
    o = pb.softmax_attention(q, k, v, np.arange(T), 1.0, chunk=4)
    assert np.allclose(o[3, 0], (1 + 2 + 3 + 4) / 4) and np.allclose(o[4, 1], 5.0) and np.allclose(o[5, 0], 5.5)
    o = pb.softmax_attention(q, k, v, np.arange(T), 1.0, chunk=4, sink=True)
    assert np.allclose(o[3, 0], 10 / 5) and np.allclose(o[4, 0], 5 / 2)
    o = pb.softmax_attention(q, k, v, np.arange(T), 1.0)
    assert np.allclose(o[5, 1], 3.5)
    # two key heads: query heads 0, 1 read the first, 2, 3 the second
    k2 = np.zeros((T, 2, d))
    v2 = np.stack([np.ones((T, 1)), 2 * np.ones((T, 1))], axis=1)
    o = pb.softmax_attention(np.zeros((T, 4, d)), k2, v2, np.arange(T), 1.0)
    assert np.allclose(o[:, :2], 1.0) and np.allclose(o[:, 2:], 2.0)


def test_lightning_attention_in_closed_form_for_two_tokens():
    m = {"heads": 1, "dim": 2, "vdim": 1, "decay": [0.5]}
    eye = np.eye(2)
    w = {"m.q": eye, "m.k": eye, "m.v": np.array([[1.0, 0.0]]), "m.g": np.zeros((1, 2)), "m.norm": np.ones(1),
         "m.o": np.ones((2, 1))}
    h = np.array([[1.0, 2.0], [3.0, -1.0]])
    s = pb.silu(h)
    S1 = np.outer(s[0], s[0, :1])
    S2 = 0.5 * S1 + np.outer(s[1], s[1, :1])
    o = np.array([[S1[:, 0] @ s[0]], [S2[:, 0] @ s[1]]])
    want = (o / np.sqrt(o * o + 1e-6)) * 0.5                        # norm over one column, gate sigmoid(0)
    got, S = pb.lightning(h, w, "m.", m, 1e-6)
    assert np.allclose(got, want @ np.ones((1, 2))) and np.allclose(S[0], S2)
    # a state carried over equals the whole
    a, Sa = pb.lightning(h[:1], w, "m.", m, 1e-6)
    b, _ = pb.lightning(h[1:], w, "m.", m, 1e-6, Sa)
    assert np.allclose(np.concatenate([a, b]), got)


def test_the_gated_recurrence_in_closed_form_and_its_convolution_over_a_cut():
    m = {"width": 2, "conv": 2, "blocks": 2}
    w = {"m.y": np.eye(2), "m.y.b": np.zeros(2), "m.x": np.eye(2), "m.x.b": np.array([0.5, 0.0]),
         "m.conv": np.array([[2.0, 1.0], [0.0, 1.0]]), "m.conv.b": np.array([0.0, 0.25]),
         "m.ra": np.zeros((2, 1, 1)), "m.ra.b": np.zeros((2, 1)), "m.ri": np.zeros((2, 1, 1)), "m.ri.b": np.zeros((2, 1)),
         "m.lam": np.zeros(2), "m.o": np.eye(2)}
    h = np.array([[1.0, 2.0], [3.0, 4.0]])
    xin = h + np.array([0.5, 0.0])
    u = np.array([[xin[0, 0], xin[0, 1] + 0.25], [2 * xin[0, 0] + xin[1, 0], xin[1, 1] + 0.25]])   # zeros before the start
    a = math.exp(-8 * 0.5 * math.log(2.0))
    b = math.sqrt(1 - a * a) * 0.5
    S1 = b * u[0]
    S2 = a * S1 + b * u[1]
    want = np.stack([S1, S2]) * pb.gelu_tanh(h)
    got, st = pb.gated_linear_recurrence(h, w, "m.", m)
    assert np.allclose(got, want) and np.allclose(st[1], S2) and np.allclose(st[0], xin[1:])
    first, st1 = pb.gated_linear_recurrence(h[:1], w, "m.", m)
    second, _ = pb.gated_linear_recurrence(h[1:], w, "m.", m, st1)
    assert np.allclose(np.concatenate([first, second]), got)
    assert abs(pb.gelu_tanh(np.array([1.0]))[0] - 0.8411919906082768) < 1e-12


def test_copies_of_the_stream_with_an_identity_mix_are_the_plain_residual():
    cfg = copy.deepcopy(BAF_C)
    g = np.random.default_rng(1)
    shapes = _shapes(cfg)
    w = {n: g.standard_normal(s) * (0.3 if len(s) > 1 else 0.1) for n, s in shapes.items()}
    toks = g.integers(0, cfg["vocab"], 9)
    want, _ = pb.forward(toks, w, cfg)
    cfg2 = copy.deepcopy(cfg)
    cfg2["streams"] = 3
    w2 = dict(w)
    for i, l in enumerate(cfg["layers"]):
        for q in (1, 2) if l["mlp"] else (1,):
            # reading the first copy and writing it alone is the plain residual; the other copies carry rubbish along
            w2[f"l{i}.hc{q}.in"] = np.array([1.0, 0.0, 0.0])
            w2[f"l{i}.hc{q}.mix"] = np.array([[1.0, 0.3, 0.0], [0.0, 0.5, 0.2], [0.0, 0.1, 0.7]])
            w2[f"l{i}.hc{q}.out"] = np.array([1.0, -2.0, 0.5])
    got, seen = pb.forward(toks, w2, cfg2)
    assert not np.allclose(got, want)            # the output sums all copies
    w2 = {k: (v * np.array([1.0, 0.0, 0.0]) if k.endswith(".out") and ".hc" in k else v) for k, v in w2.items()}
    for k in list(w2):
        if k.endswith(".mix") and ".hc" in k:
            w2[k] = np.array([[1.0, 0.0, 0.0], [0.0, 0.0, 0.0], [0.0, 0.0, 0.0]])
    got, _ = pb.forward(toks, w2, cfg2)
    # the two copies that start as the embedding's rows vanish at the first update: only the first is left in the sum
    assert np.allclose(got, want)


def test_the_loop_runs_its_layers_in_a_row_and_the_rest_behind():
    assert pb.run_order({"layers": [0] * 4, "loop": {"start": 1, "stop": 3, "times": 2}}) == [0, 1, 2, 1, 2, 3]
    assert pb.run_order({"layers": [0] * 2}) == [0, 1]


def _shapes(cfg):
    """Tensor names and shapes of a configuration, from the engine's own declaration of them."""
    from atoma_infer_amd.config.registry import resolve_architecture
    from atoma_infer_amd.weights.loader import expected_tensors
    arch = resolve_architecture(cfg)
    return {n: ws.drawn_shape for n, ws in expected_tensors(arch.build(arch.config_cls.from_dict(cfg))).items()}


# ---- configuration and builder -----------------------------------------------------------------------------------

@pytest.mark.parametrize("cfg", [BAF_A, BAF_B, BAF_C, BAF_D])
def test_a_configuration_reads_back_equal_and_declares_its_tensors(cfg):
    from atoma_infer_amd.config.bafilorn import BafilornConfig
    c = BafilornConfig.from_dict(copy.deepcopy(cfg))
    assert BafilornConfig.from_dict(c.to_dict()) == c
    shapes = _shapes(cfg)
    s = cfg.get("streams")
    for i, l in enumerate(cfg["layers"]):
        assert (f"l{i}.hc1.mix" in shapes) == (s is not None) and (f"l{i}.norm2" in shapes) == (l["mlp"] is not None)
        assert (f"l{i}.hc2.in" in shapes) == (s is not None and l["mlp"] is not None)
        if s is not None:
            assert shapes[f"l{i}.hc1.mix"] == (s, s) and shapes[f"l{i}.hc1.out"] == (s,)
        if l["type"] == "parallel":
            m = l["mixer"]
            assert shapes[f"l{i}.mix.left.k"] == (m["left"]["kv_heads"] * m["left"]["dim"], cfg["width"])
            assert shapes[f"l{i}.mix.right.ra"] == (m["right"]["blocks"],) + (m["right"]["width"] // m["right"]["blocks"],) * 2
            assert shapes[f"l{i}.mix.left.out"] == shapes[f"l{i}.mix.right.out"] == (cfg["width"],)
            assert f"l{i}.mix.left.v" not in shapes
        if l["type"] == "latent_attention":
            m = l["mixer"]
            assert shapes[f"l{i}.mix.dkv"] == (m["kv_rank"] + m["rot_dim"], cfg["width"])
            assert shapes[f"l{i}.mix.uq"] == (m["heads"] * (m["dim"] + m["rot_dim"]), m["q_rank"])
    bg = cfg["embedding"].get("bigram")
    assert ("bigram" in shapes) == (bg is not None)
    if bg:
        assert shapes["bigram"] == (bg["buckets"] + 1, cfg["width"])


def test_the_run_order_gives_every_pass_a_call_of_its_own_and_states_are_planned_per_call():
    from atoma_infer_amd.cache.pool import EMBEDDING_CALL, plan_cache
    from atoma_infer_amd.config.registry import resolve_architecture
    arch = resolve_architecture(BAF_A)
    spec = arch.build(arch.config_cls.from_dict(copy.deepcopy(BAF_A)))
    assert [c.layer for c in spec.run_order] == [0, 1, 2, 1, 2]
    plan = plan_cache(spec)
    # the pair table's previous token, the lightning layer's S, and the recurrence of both passes of the parallel layer
    assert plan.states[EMBEDDING_CALL] == ((1,), "int32")
    assert set(plan.states) == {EMBEDDING_CALL, 0, 1, 3}
    # two groups of pages (chunked attention, latent attention), two calls in each
    assert sorted(len(g.calls) for g in plan.groups) == [2, 2]
    assert sorted((g.spec.chunk or 0) for g in plan.groups) == [0, 7]
    none = resolve_architecture(BAF_B)
    assert EMBEDDING_CALL not in plan_cache(none.build(none.config_cls.from_dict(copy.deepcopy(BAF_B)))).states


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][1]["mixer"]["left"].update(vdim=16), "values are the keys"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(blocks=5), "does not divide"),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5]), "decays for"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=10), "cannot hold"),
    (lambda c: c["layers"][2]["mixer"].update(kv_rank=300), "more than the attention kernels"),
    (lambda c: c.update(loop={"start": 2, "stop": 5, "times": 2}), "does not lie within"),
    (lambda c: c.update(streams=9), "more than 8 copies"),
    (lambda c: c["layers"][0].update(type="convolution"), "is not supported"),
])
def test_a_configuration_the_engine_cannot_run_is_refused_with_the_reason(change, message):
    from atoma_infer_amd.config.base import ConfigError
    from atoma_infer_amd.config.bafilorn import BafilornConfig
    c = copy.deepcopy(BAF_A)
    change(c)
    with pytest.raises(ConfigError, match=message):
        BafilornConfig.from_dict(c)
