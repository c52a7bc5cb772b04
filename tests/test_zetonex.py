"""Zetonex on the CPU: the plain implementation's mechanisms pinned to independent facts, the configuration
reader, the tensor names, the order in which the layers run and what the model asks of the cache manager."""
from __future__ import annotations

import copy
import math

import pytest
import torch

import plain_zetonex as plain
import zetonex_models as zm

F64 = torch.float64


def _rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def test_centered_norm_is_the_plain_norm_with_one_added():
    x, w = _rand(5, 12), _rand(12, seed=1) * 0.1
    assert torch.allclose(plain.norm_centered(x, w, 1e-5), plain.norm_plain(x, w + 1.0, 1e-5))
    unit = plain.norm_plain(x, torch.ones(12, dtype=F64), 0.0)
    assert torch.allclose((unit * unit).mean(-1), torch.ones(5, dtype=F64))


def test_rotation_turns_halves_and_depends_on_distance():
    rot = {"dims": 8, "base": 50.0}
    q, k = _rand(1, 12), _rand(1, 12, seed=1)

    def score(pq, pk):
        return float((plain.rotate_halves(q, torch.tensor([pq]), rot) * plain.rotate_halves(k, torch.tensor([pk]), rot)).sum())

    assert score(7, 3) == pytest.approx(score(104, 100), rel=1e-9)
    assert score(0, 0) == pytest.approx(float((q * k).sum()), rel=1e-12)
    assert abs(score(7, 3) - score(7, 4)) > 1e-3
    # entry i turns with entry i + dims / 2; entries behind dims stay
    x = torch.zeros(1, 12, dtype=F64)
    x[0, 1] = 1.0
    x[0, 10] = 2.0
    y = plain.rotate_halves(x, torch.tensor([5]), rot)
    assert sorted(torch.nonzero(y[0]).flatten().tolist()) == [1, 5, 10] and y[0, 10] == 2.0
    ang = 5 * 50.0 ** (-2.0 / 8)
    assert y[0, 1] == pytest.approx(math.cos(ang)) and y[0, 5] == pytest.approx(math.sin(ang))


def test_frequency_bands():
    f = plain.frequencies({"dims": 16, "base": 100.0})
    assert torch.allclose(f, 100.0 ** (-torch.arange(8, dtype=F64) / 8))
    sc = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    g = plain.frequencies({"dims": 16, "base": 100.0, "scaling": sc})
    wave = 2 * math.pi / f
    for i in range(8):
        if wave[i] < 16:
            assert g[i] == f[i]
        elif wave[i] > 64:
            assert g[i] == pytest.approx(float(f[i]) / 8.0)
        else:
            assert f[i] / 8.0 <= g[i] <= f[i]
    assert any(16 <= w <= 64 for w in wave) and any(w > 64 for w in wave) and any(w < 16 for w in wave)
    # the engine's frequencies are the same numbers
    from llmengine.parts.window_attention import banded_frequencies
    assert torch.allclose(banded_frequencies(16, 100.0, sc), g, rtol=1e-14)
    assert torch.allclose(banded_frequencies(16, 100.0, None), f, rtol=1e-14)


def test_who_sees_whom():
    m = plain.visible(12, 4, 2)
    assert m[11].tolist() == [True, True] + [False] * 6 + [True] * 4
    assert m[3].tolist() == [True] * 4 + [False] * 8 and m[0].tolist() == [True] + [False] * 11
    assert plain.visible(6).tolist() == torch.tril(torch.ones(6, 6, dtype=torch.bool)).tolist()
    assert plain.visible(9, 1)[8].tolist() == [False] * 8 + [True]
    # a window that keeps nothing: exactly `size` keys, the token itself among them
    assert int(plain.visible(30, 7)[29].sum()) == 7 and int(plain.visible(30, 7, 3)[29].sum()) == 10


def test_one_head_of_the_gated_attention_by_hand():
    m = {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 0.7, "mask": {"size": 2, "keep_first": 1}}
    w = {"q": _rand(4, 6), "k": _rand(4, 6, seed=1), "g": _rand(4, 6, seed=2), "o": _rand(6, 4, seed=3)}
    x = _rand(4, 6, seed=4)
    q, k = x @ w["q"].T, x @ w["k"].T
    t = 3                                           # sees keys 0 (kept), 2 and 3
    s = torch.tensor([float(q[t] @ k[j]) * 0.7 for j in (0, 2, 3)], dtype=F64)
    p = torch.softmax(s, 0)
    o = p[0] * k[0] + p[1] * k[2] + p[2] * k[3]     # the values are the keys
    want = (o * torch.sigmoid(x[t] @ w["g"].T)) @ w["o"].T
    assert torch.allclose(plain.gated_attention(x, w, m)[t], want, rtol=1e-10)


def test_the_differential_attention_takes_the_second_map_off_the_first():
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 6, "scale": 0.5, "diff": 0.25, "softcap": 3.0, "mask": {"size": 3}}
    w = {"q": _rand(16, 5), "k": _rand(8, 5, seed=1), "v": _rand(6, 5, seed=2), "o": _rand(5, 12, seed=3),
         "q.norm": _rand(4, seed=4), "k.norm": _rand(4, seed=5), "lq1": _rand(4, seed=6) * 0.3, "lk1": _rand(4, seed=7) * 0.3,
         "lq2": _rand(4, seed=8) * 0.3, "lk2": _rand(4, seed=9) * 0.3}
    x = _rand(7, 5, seed=10)
    lam = plain.differential_lambda(w, 0.25)
    assert lam == pytest.approx(math.exp(float(w["lq1"] @ w["lk1"])) - math.exp(float(w["lq2"] @ w["lk2"])) + 0.25)
    got = plain.differential_attention(x, w, m, 1e-6)
    # by hand: token 5, head 1 (rows 8..15 of q: map 1 then map 2), keys 3..5
    t, eps = 5, 1e-6
    unit = lambda z: z / math.sqrt(float((z * z).mean()) + eps)
    qs = x[t] @ w["q"].T
    ks, vs = x @ w["k"].T, x @ w["v"].T
    outs = []
    for mp in range(2):
        q = unit(qs[8 + 4 * mp: 12 + 4 * mp]) * w["q.norm"]
        s = []
        for j in (3, 4, 5):
            k = unit(ks[j, 4 * mp: 4 * mp + 4]) * w["k.norm"]
            s.append(3.0 * math.tanh(float(q @ k) * 0.5 / 3.0))
        p = torch.softmax(torch.tensor(s, dtype=F64), 0)
        outs.append(p[0] * vs[3] + p[1] * vs[4] + p[2] * vs[5])
    o1 = unit(outs[0] - lam * outs[1]) * 0.75
    # head 0 the same way is not needed: put zeros there through the output matrix's columns
    wo = w["o"].clone()
    wo[:, :6] = 0
    only = plain.differential_attention(x, {**w, "o": wo}, m, eps)[t]
    assert torch.allclose(only, o1 @ wo[:, 6:].T, rtol=1e-9)
    assert got.shape == (7, 5)


def test_experts_by_table_and_their_clamps():
    mlp = {"kind": "moe", "router": {"experts": 3, "top": 2}, "expert": {"ff": 4, "limit": 0.5}}
    w = {}
    for e in range(3):
        w.update({f"e{e}.gate": _rand(4, 5, seed=e), f"e{e}.up": _rand(4, 5, seed=10 + e), f"e{e}.down": _rand(5, 4, seed=20 + e)})
    w["table"] = torch.tensor([[0, 2], [1, 0], [2, 1]], dtype=torch.int32)
    x = _rand(3, 5, seed=30) * 2
    got = plain.table_experts(x, [1, 1, 2], w, mlp)
    assert torch.allclose(got[0] + 0, (plain.expert_ff(x[:1], w, 1, 0.5)[0] + plain.expert_ff(x[:1], w, 0, 0.5)[0]) / 2)
    # the gate is clamped from above only, the up value on both sides; the up value has one added
    g, u = x[2] @ w["e2.gate"].T, x[2] @ w["e2.up"].T
    assert (g > 0.5).any() or (u.abs() > 0.5).any()
    g, u = g.clamp(max=0.5), u.clamp(-0.5, 0.5)
    assert torch.allclose(plain.expert_ff(x[2:3], w, 2, 0.5)[0], (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w["e2.down"].T)


def test_the_order_of_layers_and_passes():
    assert plain.layer_order({"layers": [0] * 4}) == [(i, False) for i in range(4)]
    assert plain.layer_order({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 2}}) == \
        [(0, False), (1, True), (2, False), (1, True), (2, False), (3, False), (4, False)]
    from llmengine.config import parse_config, resolve
    for cfg in (zm.MIXED, zm.ALIGNED, zm.config([zm.gated()], loop=(0, 1, 1)), zm.config([zm.gated(), zm.differential()])):
        c = parse_config(cfg)
        model = resolve("Zetonex").build_model(c)
        assert [(call.layer, call.enter) for call in model.schedule] == plain.layer_order(cfg)
        ids = [call.cache_id for call in model.schedule]
        assert len(set(ids)) == len(ids)                # every run of a layer has a cache of its own
        assert (model.pass_input is not None) == ("loop" in cfg)


def test_config_reader_names_and_refusals():
    from llmengine.config import ConfigError, parse_config, resolve
    c = parse_config(zm.MIXED)
    assert c.architecture == "Zetonex" and c.width == 28 and c.loop == (1, 3, 2) and c.logit_scale == 1.5
    assert c.layers[1].mixer["keep_first"] == 3 and c.layers[1].mixer["window"] == 9 and c.layers[4].mixer["rot"]["dims"] == 0
    model = resolve("Zetonex").build_model(c)
    names = model.named_specs()
    for n in ("embed", "loop.in", "l0.norm1", "l0.mix.q", "l0.mix.q.norm", "l0.mix.lk2", "l0.mlp.gate.b", "l0.mlp.down.b", "l1.mix.g",
              "l3.mlp.e2.down", "l3.mlp.table", "final.norm", "head"):
        assert n in names, n
    assert "l1.mix.v" not in names and "l2.mlp.gate" not in names and "l0.mix.g" not in names and "l3.mlp.router" not in names
    assert tuple(names["loop.in"].shape) == (28, 56) and tuple(names["l0.mix.q"].shape) == (2 * 2 * 10, 28)
    assert tuple(names["l0.mix.k"].shape) == (1 * 2 * 10, 28) and tuple(names["l3.mlp.table"].shape) == (61, 1)
    bad = copy.deepcopy(zm.MIXED)
    bad["layers"][1]["mixer"]["vdim"] = 10
    with pytest.raises(ConfigError, match="vdim"):
        parse_config(bad)
    bad = copy.deepcopy(zm.MIXED)
    bad["loop"]["stop"] = 9
    with pytest.raises(ConfigError, match="stop"):
        parse_config(bad)
    bad = copy.deepcopy(zm.MIXED)
    bad["layers"][0]["type"] = "attention_3"
    with pytest.raises(ConfigError, match="attention_3"):
        parse_config(bad)
    bad = copy.deepcopy(zm.MIXED)
    bad["layers"][3]["mlp"]["router"]["top"] = 4
    with pytest.raises(ConfigError, match="top"):
        parse_config(bad)


def test_cache_specs_follow_the_masks():
    from llmengine.config import parse_config, resolve
    model = resolve("Zetonex").build_model(parse_config(zm.MIXED))
    specs = model.cache_specs()
    by_layer = {call.layer: specs[call.cache_id] for call in model.schedule}
    assert (by_layer[0].kind, by_layer[0].window) == ("window", 11)
    assert by_layer[1].kind == "full"                               # kept first tokens stay in their pages
    assert (by_layer[3].kind, by_layer[3].window) == ("window", 13)  # the same mixer with nothing kept slides
    assert tuple(by_layer[0].paged["k"]) == (2, -1, 10) and tuple(by_layer[0].paged["v"]) == (1, 14, -1)
    assert tuple(by_layer[1].paged["k"]) == (2, -1, 12) and tuple(by_layer[1].paged["v"]) == (2, 12, -1)
    assert len(specs) == 7


def test_random_weights_of_the_design(tmp_path):
    from llmengine.weights import write_random_model
    from safetensors import safe_open
    folder = write_random_model(zm.MIXED, str(tmp_path), 5)
    with safe_open(f"{folder}/model.safetensors", "pt") as f:
        table = f.get_tensor("l3.mlp.table")
        assert table.dtype == torch.int32 and int(table.min()) >= 0 and int(table.max()) < 3
        assert f.get_tensor("l0.mlp.gate.b").dtype == torch.bfloat16
    cfg = zm.config([zm.gated(mlp=zm.feed_forward("moe", experts=6, top=3))])
    folder = write_random_model(cfg, str(tmp_path / "b"), 6)
    with safe_open(f"{folder}/model.safetensors", "pt") as f:
        table = f.get_tensor("l0.mlp.table")
        assert all(len(set(row.tolist())) == 3 for row in table)


def test_the_sharp_test_weights_show_a_window_that_is_one_off():
    """The GPU tests rely on this: with the scales multiplied, a window one token longer, one kept token more or a
    cap left out moves the plain model's logits far beyond the tolerances."""
    cfg = zm.config([zm.gated(window=9, keep_first=3, sharp=6.0, mlp=None), zm.differential(window=7, softcap=4.0, sharp=6.0, mlp=None)])
    w = {k: v.float() for k, v in zm.make_weights(cfg, 3, torch.float32).items()}
    ids = torch.randint(0, cfg["vocab"], (60,), generator=torch.Generator().manual_seed(1)).tolist()
    base = plain.forward(cfg, w, ids)
    rel = lambda other: float(((other - base) ** 2).mean().sqrt() / (base ** 2).mean().sqrt())
    for path, value in ((("layers", 0, "mixer", "mask", "size"), 10), (("layers", 0, "mixer", "mask", "keep_first"), 4),
                        (("layers", 1, "mixer", "mask", "size"), 6), (("layers", 1, "mixer", "softcap"), 0.0)):
        other = copy.deepcopy(cfg)
        node = other
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        assert rel(plain.forward(other, w, ids)) > 3e-2, path
