"""Rakuvik without a GPU: the configuration, the builder's tensor names, the random-weights mode, and what pins the
plain implementation (closed forms worked out by hand)."""
import copy
import math

import pytest
import torch

import plain_rakuvik as pr
from rakuvik_util import RAK_A, RAK_B, RAK_C, RAK_D, attention, config, dense, layer, mingru, moe


def _spec(cfg):
    from atoma_infer_amd.config.registry import resolve_architecture
    arch = resolve_architecture(cfg)
    c = arch.config_cls.from_dict(copy.deepcopy(cfg))
    return arch, c, arch.build(c)


@pytest.mark.parametrize("cfg", [RAK_A, RAK_B, RAK_C, RAK_D])
def test_configuration_reads_back_and_the_builder_names_the_checkpoint_s_tensors(cfg):
    from atoma_infer_amd.weights.loader import expected_tensors
    arch, c, spec = _spec(cfg)
    assert arch.name == "Rakuvik" and c.to_dict() == cfg
    names = expected_tensors(spec)
    assert names["embed"].shape == (cfg["vocab"], cfg["width"]) and names["final.norm"].shape == ()
    for i, l in enumerate(cfg["layers"]):
        m = l["mixer"]
        assert names[f"l{i}.norm1"].shape == () and names[f"l{i}.dwa"].shape == (i + 2,)
        assert (f"l{i}.norm2" in names) == (l["mlp"] is not None)
        if l["type"] == "attention":
            assert names[f"l{i}.mix.q"].shape == (m["heads"] * 2 * m["dim"], cfg["width"])
            assert names[f"l{i}.mix.g"].shape == (m["heads"], cfg["width"])
            assert names[f"l{i}.mix.o"].shape == (cfg["width"], m["heads"] * m["vdim"])
            assert names[f"l{i}.mix.lk2"].shape == (m["dim"],)
            assert (f"l{i}.mix.k" in names) == (f"l{i}.mix.v" in names) == ("kv_from" not in m)
            if "kv_from" not in m:
                assert names[f"l{i}.mix.k"].shape == (m["kv_heads"] * 2 * m["dim"], cfg["width"])
                assert names[f"l{i}.mix.v"].shape == (m["kv_heads"] * m["vdim"], cfg["width"])
        else:
            assert names[f"l{i}.mix.z.b"].shape == (m["width"],) and names[f"l{i}.mix.o"].shape == (cfg["width"], m["width"])
        if l["mlp"] and l["mlp"]["kind"] == "moe":
            r = l["mlp"]["router"]
            assert names[f"l{i}.mlp.router"].shape == (r["experts"], cfg["width"])
            assert names[f"l{i}.mlp.correction"].shape == (r["experts"],)
            assert names[f"l{i}.mlp.e{r['experts'] - 1}.down"].shape == (cfg["width"], l["mlp"]["expert"]["ff"])
            assert f"l{i}.mlp.e0.gate" not in names
            assert (f"l{i}.mlp.shared.sg" in names) == ("shared" in l["mlp"])
        elif l["mlp"]:
            assert names[f"l{i}.mlp.gate"].shape == (l["mlp"]["ff"], cfg["width"])


def test_a_layer_that_reads_another_s_cache_owns_none():
    from atoma_infer_amd.cache.pool import plan_cache
    _, _, spec = _spec(RAK_B)
    assert [c.kv_from for c in spec.run_order] == [None, None, 0, None, 0]
    plan = plan_cache(spec)
    assert plan.where[2][:2] == plan.where[0][:2] == plan.where[4][:2]
    assert plan.where[0][2] and not plan.where[2][2] and not plan.where[4][2]
    assert plan.where[3][0] != plan.where[0][0]            # other sizes: a group of pages of its own
    assert set(plan.states) == {1} and plan.states[1][0] == (192,)
    # one key of both maps' columns and the values once: 2 x 32 and 64 columns a head
    assert plan.groups[plan.where[0][0]].spec.head_size == 64 and plan.groups[plan.where[3][0]].spec.head_size == 128


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=18), "rotated columns"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=0), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=8), "cache it reads"),
    (lambda c: c["layers"][0].update(type="gru"), "not supported"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "kind"),
    (lambda c: c["layers"][3]["mlp"]["router"].update(top=9), "exceeds"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_configurations_that_cannot_run_are_refused(change, text):
    from atoma_infer_amd.config.base import ConfigError
    cfg = copy.deepcopy(RAK_A)
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        _spec(cfg)


def test_random_weights_load_back(tmp_path):
    from safetensors.torch import load_file
    from atoma_infer_amd.weights import write_random_model
    d = write_random_model(str(tmp_path / "m"), copy.deepcopy(RAK_A), seed=3, dtype="bfloat16", norm_jitter=0.1)
    w = load_file(d + "/model.safetensors")
    assert w["l0.norm1"].shape == () and w["l3.dwa"].shape == (5,) and float(w["l3.dwa"][-1]) > 0.4
    logits = pr.forward([5, 9, 2, 77, 1], {k: v for k, v in w.items()}, RAK_A)
    assert logits.shape == (5, 97) and bool(torch.isfinite(logits).all())


def test_stretches_of_a_step_cover_every_token_once_in_order():
    from atoma_infer_amd.kernels.ops import MINGRU_STRETCH_MIN_TOKENS, mingru_plan
    assert mingru_plan([1, 1, MINGRU_STRETCH_MIN_TOKENS - 1], 64) is None
    for counts, width in (([300, 1, 17], 64), ([64], 4096), ([5000, 2, 2, 700], 2048)):
        arr, n = mingru_plan(counts, width)
        rows, first = arr[: 3 * n].reshape(n, 3), arr[3 * n:]
        assert len(first) == len(counts) + 1 and first[0] == 0 and first[-1] == n
        at = 0
        for e, c in enumerate(counts):
            mine = rows[first[e]: first[e + 1]]
            assert (mine[:, 0] == e).all() and mine[0, 1] == at and mine[-1, 2] == at + c
            assert (mine[1:, 1] == mine[:-1, 2]).all() and (mine[:, 2] > mine[:, 1]).all()
            at += c


# ---- what pins the plain implementation ------------------------------------------------------------------------------

def test_plain_norm_and_activations():
    x = torch.tensor([[3.0, -4.0]], dtype=torch.float64)
    g = torch.tensor(2.0, dtype=torch.float64)
    assert torch.allclose(pr.scalar_norm(x, g, 0.5), x / math.sqrt(12.5 + 0.5) * 2.0)
    z = torch.tensor([0.0, 1.0, -2.0], dtype=torch.float64)
    want = [0.0, 0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * 1.044715)),
            -1.0 * (1 + math.tanh(math.sqrt(2 / math.pi) * (-2 - 0.044715 * 8)))]
    assert torch.allclose(pr.gelu_tanh(z), torch.tensor(want, dtype=torch.float64))


def test_plain_frequencies_and_rotation_pairs_signs_and_shift():
    f = pr.linear_scaled_frequencies(100.0, 4, 4.0)
    assert torch.allclose(f, torch.tensor([1.0 / 4, 0.1 / 4], dtype=torch.float64))
    x = torch.zeros(1, 1, 6, dtype=torch.float64)
    x[0, 0] = torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0])
    y = pr.rotate_halves(x, torch.tensor([2]), f)
    a, b = 2 * 0.25, 2 * 0.025
    want = [math.cos(a) - 3 * math.sin(a), 2 * math.cos(b) - 4 * math.sin(b), 3 * math.cos(a) + math.sin(a),
            4 * math.cos(b) + 2 * math.sin(b), 5.0, 6.0]                  # pairs (0, 2) and (1, 3); the rest passes
    assert torch.allclose(y[0, 0], torch.tensor(want, dtype=torch.float64))
    # scores depend on the distance of the positions only
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 1, 4, generator=g, dtype=torch.float64), torch.randn(1, 1, 4, generator=g, dtype=torch.float64)
    s = [float((pr.rotate_halves(q, torch.tensor([p + 3]), f) * pr.rotate_halves(k, torch.tensor([p]), f)).sum())
         for p in (0, 11)]
    assert abs(s[0] - s[1]) < 1e-12


def _attention_weights(m, width, seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    return {"a.q": r(m["heads"] * 2 * m["dim"], width), "a.k": r(m["kv_heads"] * 2 * m["dim"], width),
            "a.v": r(m["kv_heads"] * m["vdim"], width), "a.g": r(m["heads"], width),
            "a.o": r(width, m["heads"] * m["vdim"]), "a.lq1": r(m["dim"]) * 0.3, "a.lk1": r(m["dim"]) * 0.3,
            "a.lq2": r(m["dim"]) * 0.3, "a.lk2": r(m["dim"]) * 0.3}


def test_plain_differential_attention_one_and_two_tokens_by_hand():
    """One token: both maps put all weight on it, o = (1 - lam) v.  Two tokens, one head, no rotation: the second
    row's weights are worked out with exp by hand for both maps."""
    m = attention(dim=2, heads=1, kv_heads=1, vdim=3, scale=0.5, diff=0.25, rot_dims=None)
    w = _attention_weights(m, 4)
    h = torch.randn(2, 4, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    lam = math.exp(float(w["a.lq1"] @ w["a.lk1"])) - math.exp(float(w["a.lq2"] @ w["a.lk2"])) + 0.25
    assert abs(pr.difference_weight(w, "a.", m) - lam) < 1e-12
    q, k, v = h @ w["a.q"].T, h @ w["a.k"].T, h @ w["a.v"].T
    rows = []
    for t in range(2):
        maps = []
        for j in range(2):
            s = [0.5 * float(q[t, 2 * j: 2 * j + 2] @ k[u, 2 * j: 2 * j + 2]) for u in range(t + 1)]
            e = [math.exp(x) for x in s]
            maps.append(sum(p / sum(e) * v[u] for u, p in enumerate(e)))
        o = maps[0] - lam * maps[1]
        o = o / torch.sqrt((o * o).mean() + 1e-5) * 0.75
        rows.append((o * torch.sigmoid(h[t] @ w["a.g"][0])) @ w["a.o"].T)
    got = pr.differential_attention(h, w, "a.", m, 1e-5)
    assert torch.allclose(got, torch.stack(rows), atol=1e-12)
    assert torch.allclose(maps[0] * 0 + v[0] * (1 - lam), (v[0] - lam * v[0]))       # the one-token case's o


def test_plain_attention_groups_heads_and_reads_another_layer_s_cache():
    m = attention(dim=4, heads=4, kv_heads=2, vdim=6, scale=0.3, diff=0.2, rot_dims=4, base=10.0, factor=2.0)
    w = _attention_weights(m, 8, seed=2)
    g = torch.Generator().manual_seed(3)
    h, other = torch.randn(5, 8, generator=g, dtype=torch.float64), torch.randn(5, 8, generator=g, dtype=torch.float64)
    own = pr.differential_attention(h, w, "a.", m, 1e-5)
    # heads 0, 1 read key head 0 and heads 2, 3 key head 1: changing key head 1's rows leaves heads 0, 1 alone
    w2 = dict(w)
    w2["a.k"] = w["a.k"].clone()
    w2["a.k"][8:] += 1.0
    w2["a.o"] = w["a.o"].clone()
    w2["a.o"][:, 12:] = 0
    w0 = dict(w, **{"a.o": w2["a.o"]})
    assert torch.allclose(pr.differential_attention(h, w2, "a.", m, 1e-5), pr.differential_attention(h, w0, "a.", m, 1e-5))
    kv = pr.keys_and_values(other, w, "a.", m)
    borrowed = pr.differential_attention(h, w, "a.", m, 1e-5, kv=kv)
    assert not torch.allclose(borrowed, own) and torch.allclose(borrowed[0].isfinite(), torch.tensor(True))
    assert torch.allclose(pr.differential_attention(h, w, "a.", m, 1e-5, kv=pr.keys_and_values(h, w, "a.", m)), own)


def test_plain_mingru_two_tokens_by_hand():
    w = {"r.z": torch.tensor([[1.0, 0.0], [0.0, 2.0]], dtype=torch.float64), "r.z.b": torch.tensor([0.5, -0.5], dtype=torch.float64),
         "r.x": torch.tensor([[0.0, 1.0], [1.0, 0.0]], dtype=torch.float64), "r.x.b": torch.tensor([0.1, -0.2], dtype=torch.float64),
         "r.g": torch.eye(2, dtype=torch.float64), "r.o": torch.tensor([[1.0, 1.0]], dtype=torch.float64)}
    h = torch.tensor([[1.0, -1.0], [0.5, 2.0]], dtype=torch.float64)
    sg = lambda x: 1 / (1 + math.exp(-x))
    s, want = [0.0, 0.0], []
    for t in range(2):
        z = [sg(h[t, 0] + 0.5), sg(2 * h[t, 1] - 0.5)]
        u = [float(h[t, 1]) + 0.1, float(h[t, 0]) - 0.2]
        c = [x + 0.5 if x >= 0 else sg(x) for x in u]
        s = [(1 - z[i]) * s[i] + z[i] * c[i] for i in range(2)]
        want.append(sum(s[i] * float(h[t, i]) * sg(float(h[t, i])) for i in range(2)))
    got = pr.mingru(h, w, "r.", {"width": 2})
    assert torch.allclose(got[:, 0], torch.tensor(want, dtype=torch.float64), atol=1e-12)
    # a candidate of exactly zero input takes the upper branch: u = 0 gives 1/2 either way, u just below gives sigmoid
    assert abs(sg(-1e-9) - 0.5) < 1e-8


def test_plain_router_chooses_with_the_correction_and_weighs_without():
    w = {"m.router": torch.eye(3, 2, dtype=torch.float64), "m.correction": torch.tensor([0.0, 0.0, 0.9], dtype=torch.float64)}
    h = torch.tensor([[2.0, 1.0]], dtype=torch.float64)
    ids, weights = pr.route(h, w, "m.", {"top": 2, "scale": 3.0})
    e = [math.exp(2.0), math.exp(1.0), 1.0]
    s = [x / sum(e) for x in e]
    assert ids.tolist() == [[2, 0]]                      # expert 2 by its correction, though its score is the lowest
    assert torch.allclose(weights, torch.tensor([[3.0 * s[2], 3.0 * s[0]]], dtype=torch.float64))


def test_plain_experts_and_the_shared_expert_by_hand():
    mlp = moe(ff=2, experts=2, top=1, scale=2.0, shared=2)
    g = torch.Generator().manual_seed(5)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    w = {"m.router": r(2, 3), "m.correction": torch.zeros(2, dtype=torch.float64), "m.shared.up": r(2, 3),
         "m.shared.down": r(3, 2), "m.shared.sg": r(1, 3)}
    for e in range(2):
        w[f"m.e{e}.up"], w[f"m.e{e}.down"] = r(2, 3), r(3, 2)
    h = r(1, 3)
    s = torch.softmax(h @ w["m.router"].T, -1)[0]
    e = int(s.argmax())
    want = 2.0 * s[e] * (torch.relu(h @ w[f"m.e{e}.up"].T) ** 2 @ w[f"m.e{e}.down"].T)
    want = want + (torch.relu(h @ w["m.shared.up"].T) ** 2 @ w["m.shared.down"].T) * torch.sigmoid(h @ w["m.shared.sg"].T)
    assert torch.allclose(pr.moe_ff(h, w, "m.", mlp), want, atol=1e-12)


def test_plain_model_of_one_layer_by_hand_with_the_depth_average():
    """One token through one attention layer and a dense feed-forward: softmax over one key is 1, so the mixer is
    W_o (gate * unit((1 - lam) v) * (1 - diff)); the layer's result and the embedding's row are then weighed."""
    from atoma_infer_amd.weights.random_init import random_tensors
    cfg = config([layer("attention", attention(dim=4, heads=2, kv_heads=1, vdim=4, scale=0.5, diff=0.3, rot_dims=4, base=9.0),
                        dense(6))], width=8, vocab=11)
    _, _, spec = _spec(cfg)
    w = {k: v.double() for k, v in random_tensors(spec, 1, torch.float32, 0.2)}
    w["l0.dwa"] = torch.tensor([0.25, 0.5], dtype=torch.float64)
    eps, tok = 1e-5, 7
    n = lambda v, g: v / torch.sqrt((v * v).mean() + eps) * g
    x0 = w["embed"][tok]
    h = n(x0, w["l0.norm1"])
    lam = pr.difference_weight(w, "l0.mix.", cfg["layers"][0]["mixer"])
    v = h @ w["l0.mix.v"].T
    o = (1 - lam) * v
    o = o / torch.sqrt((o * o).mean() + eps) * 0.7
    gate = torch.sigmoid(h @ w["l0.mix.g"].T)
    a = torch.cat([o * gate[0], o * gate[1]]) @ w["l0.mix.o"].T
    y = x0 + n(a, w["l0.norm1b"])
    h2 = n(y, w["l0.norm2"])
    f = (pr.gelu_tanh(h2 @ w["l0.mlp.gate"].T) * (h2 @ w["l0.mlp.up"].T)) @ w["l0.mlp.down"].T
    x1 = y + n(f, w["l0.norm2b"])
    out = n(0.25 * x0 + 0.5 * x1, w["final.norm"]) @ w["head"].T
    streams = []
    got = pr.forward([tok], w, cfg, streams=streams)
    assert torch.allclose(got[0], out, atol=1e-10) and torch.allclose(streams[0][0], x1, atol=1e-10)


def test_plain_model_does_not_look_ahead():
    from atoma_infer_amd.weights.random_init import random_tensors
    _, _, spec = _spec(RAK_A)
    w = dict(random_tensors(spec, 2, torch.float32, 0.1))
    toks = [3, 14, 15, 92, 65, 35, 89, 79]
    full = pr.forward(toks, w, RAK_A)
    assert torch.allclose(pr.forward(toks[:5], w, RAK_A), full[:5], atol=1e-9)
    other = pr.forward(toks[:5] + [1, 2, 3], w, RAK_A)
    assert torch.allclose(other[:5], full[:5], atol=1e-9) and not torch.allclose(other[5:], full[5:])
