"""Zapolorn on the CPU: the plain implementation (tests/plain_zapolorn.py) pinned to independent facts, the
configuration reader, the tensor names, the cache specs and the random weights."""
from __future__ import annotations

import copy
import math

import pytest
import torch

import plain_zapolorn as plain
import zapolorn_models as zm

F64 = torch.float64


def _rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


# ---- the plain implementation's mechanisms -------------------------------------------------------------
def test_rotation_turns_neighbours_and_depends_on_distance_only():
    rot = {"base": 30.0, "dims": 6, "scaling": {"factor": 2.0}}
    x = _rand(1, 1, 8, seed=1)
    y = plain.rotate_neighbours(x, torch.tensor([7]), rot)
    f = [30.0 ** (-2.0 * c / 6) / 2.0 for c in range(3)]
    for c in range(3):
        a, b, ang = float(x[0, 0, 2 * c]), float(x[0, 0, 2 * c + 1]), 7 * f[c]
        assert abs(float(y[0, 0, 2 * c]) - (a * math.cos(ang) - b * math.sin(ang))) < 1e-12
        assert abs(float(y[0, 0, 2 * c + 1]) - (b * math.cos(ang) + a * math.sin(ang))) < 1e-12
    assert torch.equal(y[..., 6:], x[..., 6:])                       # the entries behind the rotated ones pass
    q, k = _rand(1, 1, 8, seed=2), _rand(1, 1, 8, seed=3)
    dot = lambda i, j: float((plain.rotate_neighbours(q, torch.tensor([i]), rot) * plain.rotate_neighbours(k, torch.tensor([j]), rot)).sum())
    assert abs(dot(40, 31) - dot(9, 0)) < 1e-10 and abs(dot(40, 31) - dot(40, 30)) > 1e-4
    # the factor stretches the positions: twice the factor at twice the position is the same turn
    slow = dict(rot, scaling={"factor": 4.0})
    assert torch.allclose(plain.rotate_neighbours(x, torch.tensor([14]), slow), y, atol=1e-12)
    assert torch.allclose(plain.pair_frequencies({"base": 30.0, "dims": 6}), plain.pair_frequencies(rot) * 2.0)


def test_the_queries_temperature_steps_with_the_position():
    t = plain.query_temperature(torch.arange(12), {"coef": 0.5, "every": 4})
    assert torch.allclose(t[:3], torch.ones(3, dtype=F64))                    # (p + 1) / 4 < 1
    assert abs(float(t[3]) - (1 + 0.5 * math.log(2))) < 1e-12 and float(t[6]) == float(t[3])
    assert abs(float(t[7]) - (1 + 0.5 * math.log(3))) < 1e-12 and abs(float(t[11]) - (1 + 0.5 * math.log(4))) < 1e-12
    assert torch.equal(plain.query_temperature(torch.arange(5), None), torch.ones(5, dtype=F64))


def test_slopes_halve_from_head_to_head_of_eight():
    assert torch.allclose(plain.head_slopes(8), torch.tensor([2.0 ** -(h + 1) for h in range(8)], dtype=F64))
    assert abs(float(plain.head_slopes(1)[0]) - 2.0 ** -8) < 1e-15 and abs(float(plain.head_slopes(3)[0]) - 2.0 ** (-8 / 3)) < 1e-15


def test_who_sees_whom_under_a_window():
    v = plain.visible(6, 3)
    assert v[5].tolist() == [False, False, False, True, True, True] and v[1].tolist() == [True, True, False, False, False, False]
    assert plain.visible(4).tolist() == torch.tril(torch.ones(4, 4, dtype=torch.bool)).tolist()
    assert plain.visible(4, 1).tolist() == torch.eye(4, dtype=torch.bool).tolist()


def test_one_head_with_a_sink_by_hand():
    q, k, v = _rand(3, 1, 4, seed=4), _rand(3, 1, 4, seed=5), _rand(3, 1, 2, seed=6)
    sink = torch.tensor([0.7], dtype=F64)
    out = plain.attend(q, k, v, 0.5, plain.visible(3), sinks=sink)
    for i in range(3):
        e = [math.exp(0.5 * float(q[i, 0] @ k[j, 0])) for j in range(i + 1)]
        den = sum(e) + math.exp(0.7)
        want = sum(e[j] / den * v[j, 0] for j in range(i + 1))
        assert torch.allclose(out[i, 0], want, atol=1e-12)
    # the sink takes its share and gives nothing: without it the first token's row is its own value
    assert torch.allclose(plain.attend(q, k, v, 0.5, plain.visible(3))[0, 0], v[0, 0])
    assert float((out[0, 0] / v[0, 0])[0]) < 1.0
    # a very large sink leaves nothing of the values, a very small one changes nothing
    assert plain.attend(q, k, v, 0.5, plain.visible(3), sinks=torch.tensor([60.0], dtype=F64)).abs().max() < 1e-20
    assert torch.allclose(plain.attend(q, k, v, 0.5, plain.visible(3), sinks=torch.tensor([-60.0], dtype=F64)),
                          plain.attend(q, k, v, 0.5, plain.visible(3)), atol=1e-12)


def test_the_distance_bias_by_hand_and_as_a_bias_on_keys():
    T = 5
    q, k, v = _rand(T, 2, 4, seed=7), _rand(T, 1, 4, seed=8), _rand(T, 1, 3, seed=9)
    slopes = plain.head_slopes(2)
    out = plain.attend(q, k, v, 0.4, plain.visible(T), slopes=slopes)
    for h in range(2):
        i = 4
        e = [math.exp(0.4 * float(q[i, h] @ k[j, 0]) - float(slopes[h]) * (i - j)) for j in range(i + 1)]
        want = sum(e[j] / sum(e) * v[j, 0] for j in range(i + 1))
        assert torch.allclose(out[i, h], want, atol=1e-12)
    # without a sink, taking slope (i - j) off is adding slope j (a row's constant leaves the softmax) ...
    k_aug = torch.cat([k, torch.arange(T, dtype=F64)[:, None, None]], dim=-1)
    for h in range(2):
        q_aug = torch.cat([q[:, h:h + 1] * 0.4, torch.full((T, 1, 1), float(slopes[h]), dtype=F64)], dim=-1)
        assert torch.allclose(plain.attend(q_aug, k_aug, v, 1.0, plain.visible(T))[:, 0], out[:, h], atol=1e-12)
    # ... with a sink it is not
    sink = torch.zeros(1, dtype=F64)
    with_sink = plain.attend(q[:, :1], k, v, 0.4, plain.visible(T), slopes=slopes[:1], sinks=sink)
    q_aug = torch.cat([q[:, :1] * 0.4, torch.full((T, 1, 1), float(slopes[0]), dtype=F64)], dim=-1)
    assert (plain.attend(q_aug, k_aug, v, 1.0, plain.visible(T), sinks=sink) - with_sink).abs().max() > 1e-3


def test_grouped_heads_read_the_key_head_of_their_group():
    T = 4
    q, k, v = _rand(T, 6, 3, seed=10), _rand(T, 2, 3, seed=11), _rand(T, 2, 5, seed=12)
    out = plain.attend(q, k, v, 1.0, plain.visible(T))
    for h in range(6):
        alone = plain.attend(q[:, h:h + 1], k[:, h // 3:h // 3 + 1], v[:, h // 3:h // 3 + 1], 1.0, plain.visible(T))
        assert torch.allclose(out[:, h], alone[:, 0], atol=1e-12)


def test_the_linear_recurrence_in_closed_form_and_carried_on():
    T, n, d, dv = 7, 2, 3, 4
    q, k, v = _rand(T, n, d, seed=13), _rand(T, n, d, seed=14), _rand(T, n, dv, seed=15)
    a = torch.sigmoid(_rand(1, n, d, seed=16)).expand(T, n, d)          # the same decay at every token
    out, S = plain.linear_recurrence(q, k, v, a)
    for t in (0, 3, 6):
        want = torch.zeros(n, dv, dtype=F64)
        for s in range(t + 1):
            want += torch.einsum("nd,nd,nv->nv", q[t] * a[0] ** (t - s), k[s], v[s])
        assert torch.allclose(out[t], want, atol=1e-12)
    # the state after four tokens carries the rest
    first, S4 = plain.linear_recurrence(q[:4], k[:4], v[:4], a[:4])
    rest, S7 = plain.linear_recurrence(q[4:], k[4:], v[4:], a[4:], state=S4)
    assert torch.allclose(torch.cat([first, rest]), out, atol=1e-12) and torch.allclose(S7, S, atol=1e-12)
    # a decay of one never forgets: the unnormalized causal linear attention
    ones = torch.ones(T, n, d, dtype=F64)
    keep, _ = plain.linear_recurrence(q, k, v, ones)
    want = torch.einsum("tsn,snv->tnv", torch.tril(torch.ones(T, T, dtype=F64))[:, :, None] * torch.einsum("tnd,snd->tsn", q, k), v)
    assert torch.allclose(keep, want, atol=1e-12)


def test_the_decay_is_a_sigmoid_flattened_by_tau():
    x = _rand(3, 5, seed=17)
    w = {"a1": _rand(2, 5, seed=18), "a2": _rand(6, 2, seed=19), "a2.b": _rand(6, seed=20)}
    z = (x @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    one = plain.channel_decay(x, w, {"heads": 2, "dim": 3, "tau": 1.0})
    assert torch.allclose(one.reshape(3, 6), torch.sigmoid(z), atol=1e-12)
    four = plain.channel_decay(x, w, {"heads": 2, "dim": 3, "tau": 4.0})
    assert torch.allclose(four ** 4, one, atol=1e-12) and bool((four > one).all())


def test_experts_weigh_their_input_not_their_result():
    H, FF, E = 6, 5, 4
    w = {"router": _rand(E, H, seed=21)}
    for e in range(E):
        w.update({f"e{e}.gate": _rand(FF, H, seed=30 + e), f"e{e}.up": _rand(FF, H, seed=40 + e), f"e{e}.down": _rand(H, FF, seed=50 + e)})
    x = _rand(3, H, seed=22)
    s = torch.sigmoid(x @ w["router"].T)
    every = plain.routed_experts(x, w, {"router": {"experts": E, "top": E}})
    want = sum(plain.gated_ff(s[:, e:e + 1] * x, plain.sub(w, f"e{e}.")) for e in range(E))
    assert torch.allclose(every, want, atol=1e-12)
    on_output = sum(s[:, e:e + 1] * plain.gated_ff(x, plain.sub(w, f"e{e}.")) for e in range(E))
    assert (every - on_output).abs().max() > 1e-3                           # (the activation does not pass a factor through)
    best = plain.routed_experts(x, w, {"router": {"experts": E, "top": 1}})
    for t in range(3):
        e = int(s[t].argmax())
        assert torch.allclose(best[t], plain.gated_ff(s[t, e] * x[t:t + 1], plain.sub(w, f"e{e}."))[0], atol=1e-12)
    # scores are not renormalized: two equal experts chosen together give twice one of them, not one
    w2 = {"router": w["router"][[0, 0]]}
    for part in ("gate", "up", "down"):
        w2[f"e0.{part}"] = w2[f"e1.{part}"] = w[f"e0.{part}"]
    two = plain.routed_experts(x, w2, {"router": {"experts": 2, "top": 2}})
    assert torch.allclose(two, 2 * plain.gated_ff(s[:, :1] * x, plain.sub(w2, "e0.")), atol=1e-9)
    # a shared expert runs on the input as it is
    w["shared.gate"], w["shared.up"], w["shared.down"] = _rand(3, H, seed=60), _rand(3, H, seed=61), _rand(H, 3, seed=62)
    both = plain.routed_experts(x, w, {"router": {"experts": E, "top": 1}, "shared": {"ff": 3}})
    assert torch.allclose(both - best, plain.gated_ff(x, plain.sub(w, "shared.")), atol=1e-12)


def test_a_layer_norms_behind_its_sublayers_and_a_reader_uses_the_writers_keys():
    cfg = zm.config([zm.windowed(window=4, mlp="dense"), zm.windowed(window=6, kv_from=0, mlp=None)])
    w = {k: v.double() for k, v in zm.make_weights(cfg, 1, torch.float32).items()}
    ids = [3, 9, 27, 1, 44, 8, 8, 15]
    logits, layers = plain.forward(cfg, w, ids, return_layers=True)
    eps, m0, m1 = cfg["norm"]["eps"], cfg["layers"][0]["mixer"], cfg["layers"][1]["mixer"]
    x0 = w["embed"][torch.tensor(ids)] * cfg["embedding"]["scale"]
    pos = torch.arange(len(ids))
    x = x0 + plain.norm(plain.window_attention(x0, plain.sub(w, "l0.mix."), m0, eps), w["l0.norm1"], eps)
    x = x + plain.norm(plain.gated_ff(x, plain.sub(w, "l0.mlp.")), w["l0.norm2"], eps)
    assert torch.allclose(layers[0], x, atol=1e-12)
    kv = plain.keys_values(x0, plain.sub(w, "l0.mix."), m0, eps, pos)          # made from the first layer's input
    y = x + plain.norm(plain.window_attention(x, plain.sub(w, "l1.mix."), m1, eps, pos, kv=kv), w["l1.norm1"], eps)
    assert torch.allclose(layers[1], y, atol=1e-12)
    assert torch.allclose(logits, plain.norm(y, w["final.norm"], eps) @ w["embed"].T * cfg["logit_scale"], atol=1e-12)
    # norm weights of zero switch a sublayer off
    w0 = dict(w)
    w0["l1.norm1"] = torch.zeros_like(w["l1.norm1"])
    assert torch.allclose(plain.forward(cfg, w0, ids, return_layers=True)[1][1], layers[0], atol=1e-12)


def test_sharp_weights_show_a_window_that_is_one_off():
    cfg = zm.config([zm.windowed(window=9, sharp=6.0, mlp=None)])
    w = zm.make_weights(cfg, 2, torch.float32)
    ids = torch.randint(0, cfg["vocab"], (60,), generator=torch.Generator().manual_seed(3)).tolist()
    ref = plain.forward(cfg, w, ids)
    off = copy.deepcopy(cfg)
    off["layers"][0]["mixer"]["mask"]["size"] = 10
    moved = (plain.forward(off, w, ids) - ref).norm(dim=-1) / ref.norm(dim=-1)
    assert float(moved[:9].max()) < 1e-12 and float(moved[9:].max()) > 0.05 and float(moved[9:].median()) > 1e-3


# ---- configuration, names, caches ---------------------------------------------------------------------
def _parse(cfg):
    from llmengine.config import parse_config
    return parse_config(cfg)


def test_the_reader_takes_every_size_and_constant():
    c = _parse(zm.MIXED)
    assert type(c).__name__ == "ZapolornConfig" and c.vocab_size == 61 and c.width == 28 and c.embedding_scale == 2.0
    assert c.norm_eps == 1e-5 and c.logit_scale == 0.6 and len(c.layers) == 7
    a = c.layers[0].mixer
    assert (a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["rot_dims"], a["rot_base"], a["rot_factor"], a["window"]) == \
           (6, 2, 12, 10, 8, 50.0, 2.0, 11) and a["kv_from"] is None
    assert c.layers[2].mixer["kv_from"] == 0 and c.layers[2].mlp is None and c.layers[6].mixer["window"] == 0
    p = c.layers[1].mixer
    assert p["left"]["q_temp"] == (0.4, 5) and p["right"] == {"heads": 2, "dim": 6, "vdim": 9, "tau": 3.0, "rank": 4}
    assert (p["left_scale"], p["right_scale"]) == (0.7, 1.3) and c.layers[5].mixer["left"]["q_temp"] is None
    assert c.layers[3].mlp == {"kind": "moe", "experts": 3, "top": 1, "ff": 24, "shared_ff": None}
    assert c.layers[4].mlp["shared_ff"] == 14 and c.layers[0].mlp == {"kind": "dense", "ff": 24}


@pytest.mark.parametrize("change, word", [
    (lambda c: c["layers"][0]["mixer"].update(heads=5), "heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=14), "dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=3), "dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].update(factor=0), "factor"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "kv_from"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(dim=10), "dim"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(base=51.0), "rot_base"),
    (lambda c: c["layers"][1]["mixer"].pop("right"), "right"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(tau=0), "tau"),
    (lambda c: c["layers"][1]["mixer"]["left"]["q_temp"].update(every=0), "every"),
    (lambda c: c["layers"][1].update(type="recurrent"), "recurrent"),
    (lambda c: c["layers"][3]["mlp"]["router"].update(top=4), "top"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "sparse"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.pop("vocab"), "vocab"),
])
def test_the_reader_refuses_by_key_name(change, word):
    from llmengine.config import ConfigError
    cfg = copy.deepcopy(zm.MIXED)
    change(cfg)
    with pytest.raises(ConfigError, match=word):
        _parse(cfg)


def _model(cfg):
    from llmengine.config.registry import resolve
    return resolve("Zapolorn").build_model(_parse(cfg))


def test_tensor_names_and_shapes():
    specs = _model(zm.MIXED).named_specs()
    shape = lambda n: tuple(specs[n].shape)
    assert shape("embed") == (61, 28) and shape("final.norm") == (28,) and "head" not in specs
    assert shape("l0.mix.q") == (72, 28) and shape("l0.mix.k") == (24, 28) and shape("l0.mix.v") == (20, 28)
    assert shape("l0.mix.q.norm") == (12,) and shape("l0.mix.k.norm") == (12,) and shape("l0.mix.sink") == (6,)
    assert shape("l0.mix.g") == (6, 28) and shape("l0.mix.o") == (28, 60) and shape("l0.norm2") == (28,)
    # a layer that reads another's keys has neither their matrices nor their norm, and this one no feed-forward
    assert sorted(n for n in specs if n.startswith("l2.")) == ["l2.mix.g", "l2.mix.o", "l2.mix.q", "l2.mix.q.norm", "l2.mix.sink", "l2.norm1"]
    assert shape("l1.mix.left.q") == (30, 28) and shape("l1.mix.left.k") == (10, 28) and shape("l1.mix.left.v") == (6, 28)
    assert shape("l1.mix.left.o") == (28, 18) and "l1.mix.left.sink" not in specs and "l1.mix.left.g" not in specs
    assert shape("l1.mix.right.q") == (12, 28) and shape("l1.mix.right.v") == (18, 28) and shape("l1.mix.right.g") == (18, 28)
    assert shape("l1.mix.right.a1") == (4, 28) and shape("l1.mix.right.a2") == (12, 4) and shape("l1.mix.right.a2.b") == (12,)
    assert shape("l1.mix.right.norm") == (9,) and shape("l1.mix.right.o") == (28, 18)
    assert shape("l1.mlp.router") == (5, 28) and shape("l1.mlp.e4.down") == (28, 24) and shape("l1.mlp.shared.gate") == (14, 28)
    assert "l3.mlp.shared.gate" not in specs and shape("l3.mlp.e2.up") == (24, 28)
    # without a rank in the configuration the decay's inner size is whatever the checkpoint holds
    cfg = copy.deepcopy(zm.MIXED)
    del cfg["layers"][1]["mixer"]["right"]["rank"]
    assert tuple(_model(cfg).named_specs()["l1.mix.right.a1"].shape) == (None, 28)


def test_cache_specs_follow_the_masks_and_the_readers():
    import torch as _t
    specs = _model(zm.MIXED).cache_specs()
    assert sorted(specs) == [0, 1, 3, 5]                                    # readers keep nothing of their own
    assert (specs[0].kind, specs[0].window) == ("window", 17)               # the widest window among layer 0 and its readers
    assert specs[3].kind == "full"                                          # its reader has no window
    assert dict(specs[0].paged) == {"k": (2, -1, 12), "v": (2, 10, -1)} and not specs[0].state
    assert specs[1].kind == "full" and dict(specs[1].paged) == {"left.k": (1, -1, 10), "left.v": (1, 6, -1)}
    assert dict(specs[1].state) == {"right.memory": ((2, 9, 6), _t.float32)}
    sched = _model(zm.MIXED).schedule
    assert [(c.layer, c.cache_id, c.write_cache) for c in sched] == [(0, 0, True), (1, 1, True), (2, 0, False), (3, 3, True),
                                                                     (4, 0, False), (5, 5, True), (6, 3, False)]


def test_random_weights_are_written_and_named_as_the_model_reads_them(tmp_path):
    from llmengine.weights import write_random_model
    from llmengine.weights.loader import check_names
    from llmengine.weights.safetensors_io import TensorIndex
    folder = write_random_model(zm.ALIGNED, str(tmp_path), 3)
    index = TensorIndex(folder)
    try:
        check_names(_model(zm.ALIGNED), {n: index.entry(n).shape for n in index.names()}, folder)
        assert "head" not in index.names() and "embed" in index.names()
    finally:
        index.close()
    cfg = copy.deepcopy(zm.ALIGNED)
    del cfg["layers"][0]["mixer"]["right"]["rank"]
    with pytest.raises(ValueError, match="only a checkpoint gives"):
        write_random_model(cfg, str(tmp_path / "x"), 3)
