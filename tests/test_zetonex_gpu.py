"""Zetonex on the GPU against the plain implementation (tests/plain_zetonex.py): every mechanism alone and
together, under every way of cutting requests into steps, in 32-bit and in bfloat16."""
from __future__ import annotations

import copy

import numpy as np
import pytest
import torch

import plain_zetonex as plain
import replay
import zetonex_models as zm

pytestmark = pytest.mark.gpu

F32_TOL = 2e-4          # of a row's root mean square; honest 32-bit arithmetic is at 1e-5
# bfloat16 against the unrounded plain model: narrow models with weights of order one; a fault of a kernel moves rows
# by their whole size. What a schedule changes is held tighter, against the whole prompts' rows.
BF16_MEAN, BF16_WORST, BF16_BETWEEN_SCHEDULES = 4e-2, 0.3, 4e-2


def _engine(tmp_path, cfg, seed, dtype, weights=None, **kw):
    from llmengine import Engine
    store = torch.float32 if dtype == "fp32" else torch.bfloat16
    folder, weights = zm.write_model(tmp_path, cfg, seed, store, weights)
    return Engine(folder, dtype, deterministic=True, **kw), weights


def _tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _reference(cfg, weights, requests):
    w = {k: (v.float() if v.is_floating_point() else v) for k, v in weights.items()}
    return {rid: plain.forward(cfg, w, ids).numpy() for rid, ids in requests.items()}


def _errors(got: dict, ref: dict) -> list[float]:
    return [float(np.sqrt(np.mean((row - ref[rid][pos]) ** 2)) / np.sqrt(np.mean(ref[rid][pos] ** 2)))
            for rid, rows in got.items() for pos, row in rows.items()]


def _worst(got, ref) -> float:
    return max(_errors(got, ref))


def _most(got, ref) -> float:
    return float(np.quantile(_errors(got, ref), 0.97))


def _mean(got, ref) -> float:
    return float(np.mean(_errors(got, ref)))


def _covered(got: dict, requests: dict) -> bool:
    return all(sorted(got[rid]) == list(range(len(ids))) for rid, ids in requests.items())


def _stacked(got: dict) -> dict:
    return {rid: np.stack([rows[p] for p in sorted(rows)]) for rid, rows in got.items()}


ONE_LAYER = {
    "gated": zm.config([zm.gated(mlp=None)]),
    "gated_sharp_keeps_three": zm.config([zm.gated(window=9, keep_first=3, sharp=6.0, mlp=None)]),
    "gated_keeps_more_than_its_window": zm.config([zm.gated(window=4, keep_first=11, sharp=5.0, mlp=None)]),
    "gated_no_window": zm.config([zm.gated(window=0, keep_first=0, sharp=4.0, mlp=None)]),
    "gated_window_of_one": zm.config([zm.gated(window=1, keep_first=2, mlp=None)]),
    "gated_no_rotation_one_head": zm.config([zm.gated(heads=1, kv_heads=1, dim=20, dims=0, window=17, keep_first=0, sharp=5.0, mlp=None)]),
    "gated_whole_head_rotated": zm.config([zm.gated(heads=6, kv_heads=3, dim=8, dims=8, window=8, keep_first=1, mlp=None)]),
    "gated_wide_heads": zm.config([zm.gated(heads=2, kv_heads=1, dim=136, dims=70, window=19, keep_first=2, scale=0.08, mlp=None)], width=36),
    "differential": zm.config([zm.differential(mlp=None)]),
    "differential_sharp": zm.config([zm.differential(window=17, sharp=6.0, mlp=None)]),
    "differential_small_cap": zm.config([zm.differential(window=8, softcap=1.5, sharp=5.0, mlp=None)]),
    "differential_no_cap_no_scaling": zm.config([zm.differential(softcap=0.0, scaling=None, sharp=3.0, mlp=None)]),
    "differential_heads_of_their_own": zm.config([zm.differential(heads=3, kv_heads=3, dim=6, vdim=4, dims=4, window=5, mlp=None)]),
    "differential_grouped_wide_values": zm.config([zm.differential(heads=6, kv_heads=2, dim=8, vdim=70, dims=8, window=30, mlp=None)]),
    "dense_with_biases": zm.config([zm.gated(mlp="dense")]),
    "experts_two_of_five": zm.config([zm.differential(mlp="moe")]),
    "experts_one_of_three": zm.config([zm.gated(mlp=zm.feed_forward("moe", experts=3, top=1, limit=0.6))]),
    "every_expert_chosen": zm.config([zm.gated(mlp=zm.feed_forward("moe", ff=10, experts=4, top=4, limit=2.0))]),
    "seventy_experts": zm.config([zm.differential(mlp=zm.feed_forward("moe", ff=6, experts=70, top=5))]),
    "one_layer_three_passes": zm.config([zm.gated(mlp="dense")], loop=(0, 1, 3)),
    "a_single_pass_still_has_its_input_map": zm.config([zm.differential(mlp=None), zm.gated(mlp=None)], loop=(1, 2, 1)),
    "width_of_30": zm.config([zm.gated(heads=5, kv_heads=5, dim=6, dims=2, mlp=zm.feed_forward("moe", ff=9))], width=30, vocab=33,
                             logit_scale=1.0),
}


@pytest.mark.parametrize("name", sorted(ONE_LAYER))
def test_each_mechanism_alone_whole_token_by_token_and_in_portions(tmp_path, name):
    cfg = ONE_LAYER[name]
    engine, weights = _engine(tmp_path, cfg, 3, "fp32")
    requests = {"a": _tokens(41, cfg["vocab"], 1), "b": _tokens(1, cfg["vocab"], 2)}
    ref = _reference(cfg, weights, requests)
    for steps in (replay.whole(requests), replay.tail_one_by_one(requests, tail=40), replay.portions(requests),
                  replay.portions(requests, sizes=(2,))):
        cache = engine.new_cache(replay.trace_peak_tokens(steps, 8) // 8 + 1, 8, 2)
        got = replay.run_trace(engine, cache, steps)
        assert _covered(got, requests)
        assert _worst(got, ref) < F32_TOL


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("cfg_name", ["MIXED", "ALIGNED"])
def test_every_schedule_gives_the_plain_logits(tmp_path, cfg_name, dtype):
    cfg = getattr(zm, cfg_name)
    engine, weights = _engine(tmp_path, cfg, 11, dtype)
    V = cfg["vocab"]
    requests = {"long": _tokens(150, V, 5), "one": _tokens(1, V, 6), "two": _tokens(2, V, 7), "mid": _tokens(49, V, 8),
                "page": _tokens(32, V, 9), "more": _tokens(65, V, 10)}
    ref = _reference(cfg, weights, requests)
    schedules = {
        "whole": replay.whole(requests),
        "tail": replay.tail_one_by_one(requests, tail=40),
        "portions": replay.portions(requests),
        "portions of two": replay.portions(requests, sizes=(2,)),
        "mixed": replay.mixed(requests, max_live=3, seed=1),
        "mixed, other cuts": replay.mixed(requests, max_live=2, sizes=(2, 17, 3, 31), seed=2),
    }
    first = None
    for what, steps in schedules.items():
        for page in (16, 8):
            # as many pages as the live requests need and three slots: pages and slots are used again
            cache = engine.new_cache(replay.trace_peak_tokens(steps, page) // page, page, 3)
            got = replay.run_trace(engine, cache, steps)
            assert _covered(got, requests), what
            if dtype == "fp32":
                assert _worst(got, ref) < F32_TOL, (what, page)
            else:
                assert _mean(got, ref) < BF16_MEAN and _most(got, ref) < BF16_WORST, (what, page)
                first = first or _stacked(got)
                assert _most(got, first) < BF16_BETWEEN_SCHEDULES and _mean(got, first) < BF16_BETWEEN_SCHEDULES / 2, (what, page)
            assert not cache.manager.live_requests()


MATRIX_CORES = {
    # three heads on one key/value head (a wavefront's 16 rows are 5 tokens and a third), key entries of 48 (a slab and a
    # half), values of 80, a window that ends inside blocks of keys, kept tokens that end inside a block
    "three_heads": zm.config([zm.gated(heads=3, kv_heads=1, dim=48, dims=24, window=37, keep_first=5, scale=0.12, sharp=3.0, mlp=None),
                              zm.differential(heads=3, kv_heads=1, dim=48, vdim=80, dims=48, window=45, scale=0.15, sharp=3.0, mlp=None)],
                             width=32),
    # every head with keys of its own (a tile holds one head of 16 tokens), heads of 16 and of 128
    "heads_of_their_own": zm.config([zm.gated(heads=4, kv_heads=4, dim=16, dims=16, window=50, keep_first=33, scale=0.2, sharp=3.0, mlp=None),
                                     zm.differential(heads=2, kv_heads=2, dim=128, vdim=128, dims=64, window=64, scale=0.09, sharp=3.0,
                                                     mlp=None)], width=32),
    # 24 heads on two key/value heads (a token's heads fill a tile and a half), no window, and a window of 130 with 70 kept
    "many_heads": zm.config([zm.gated(heads=24, kv_heads=2, dim=32, dims=8, window=0, keep_first=0, scale=0.15, sharp=3.0, mlp=None),
                             zm.gated(heads=8, kv_heads=1, dim=64, dims=32, window=130, keep_first=70, scale=0.1, sharp=3.0, mlp=None)],
                            width=32),
}


@pytest.mark.parametrize("name", sorted(MATRIX_CORES))
def test_the_matrix_core_attention_at_other_sizes(tmp_path, name):
    """bfloat16 on the matrix cores against the same model on the plain-precision kernels (what differs is the order of
    sums), under every schedule, and both against the plain model."""
    from llmengine.ops import KernelChoices
    cfg = MATRIX_CORES[name]
    engine, weights = _engine(tmp_path, cfg, 21, "bf16")
    slow_engine, _ = _engine(tmp_path / "plain", cfg, 21, "bf16", weights=weights, kernel_choices=KernelChoices(fast_attention=False))
    V = cfg["vocab"]
    requests = {"a": _tokens(300, V, 1), "b": _tokens(21, V, 2), "c": _tokens(1, V, 3)}
    ref = _reference(cfg, weights, requests)
    slow = _stacked(replay.run_trace(slow_engine, slow_engine.new_cache(32, 16, 3), replay.whole(requests)))
    for steps in (replay.whole(requests), replay.tail_one_by_one(requests, tail=150), replay.portions(requests, sizes=(33, 2, 64, 7, 1, 41)),
                  replay.mixed(requests, max_live=3, sizes=(50, 3, 24, 2), seed=4)):
        got = replay.run_trace(engine, engine.new_cache(replay.trace_peak_tokens(steps, 16) // 16, 16, 3), steps)
        assert _covered(got, requests)
        assert _mean(got, slow) < 1e-2 and _most(got, slow) < 3e-2
        assert _mean(got, ref) < 6e-2


@pytest.mark.parametrize("name", sorted(MATRIX_CORES))
def test_staged_blocks_of_keys_give_what_a_wavefront_alone_gives(tmp_path, name):
    """Prompts' attention with every block of keys staged once a workgroup through LDS walks the same blocks in the same
    order as the kernel in which a wavefront fetches its own: the logits agree to the last bits, whole and in portions."""
    from llmengine.ops import window
    cfg = MATRIX_CORES[name]
    engine, weights = _engine(tmp_path, cfg, 22, "bf16")
    V = cfg["vocab"]
    requests = {"a": _tokens(333, V, 5), "b": _tokens(70, V, 6), "c": _tokens(17, V, 7)}
    for steps in (replay.whole(requests), replay.portions(requests, sizes=(65, 16, 130, 23)),
                  replay.mixed(requests, max_live=3, sizes=(90, 40, 2), seed=9)):
        got = {}
        for staged in (True, False):
            window.WINDOW_MFMA_STAGED = staged
            try:
                got[staged] = _stacked(replay.run_trace(engine, engine.new_cache(replay.trace_peak_tokens(steps, 16) // 16, 16, 3), steps))
            finally:
                window.WINDOW_MFMA_STAGED = True
        for rid in requests:
            scale = float(np.sqrt(np.mean(got[False][rid] ** 2)))
            assert float(np.abs(got[True][rid] - got[False][rid]).max()) <= 1e-5 * scale


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_a_batch_of_unequal_requests_against_each_alone(tmp_path, dtype):
    cfg = zm.ALIGNED
    engine, _ = _engine(tmp_path, cfg, 12, dtype)
    V = cfg["vocab"]
    requests = {"a": _tokens(70, V, 1), "b": _tokens(3, V, 2), "c": _tokens(1, V, 3), "d": _tokens(33, V, 4)}
    alone = _stacked(replay.run_trace(engine, engine.new_cache(8, 16, 1), replay.whole(requests)))
    together = [{"step": 0, "entries": [{"id": r, "tokens": ids, "want": list(range(len(ids)))} for r, ids in requests.items()],
                 "end": list(requests)}]
    got = replay.run_trace(engine, engine.new_cache(12, 16, 4), together)
    assert _worst(got, alone) < (1e-5 if dtype == "fp32" else 2e-2)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_far_keys_page_borders_window_edges_and_kept_tokens(tmp_path, dtype):
    """Sharp softmaxes over a long prompt: the layer without a window finds its keys anywhere among hundreds, the windowed
    layers stand on keys just inside their windows (40 and 24 tokens: edges inside pages, at page borders and across them
    as the prompt moves along) and on the six kept tokens hundreds of positions back, in prompts cut anywhere and in
    decoding far behind the window's first pass."""
    cfg = copy.deepcopy(zm.ALIGNED)
    for layer, sharp in zip(cfg["layers"], (3.5, 3.5, 3.0)):
        layer["mixer"]["scale"] *= sharp
    engine, weights = _engine(tmp_path, cfg, 13, dtype)
    V = cfg["vocab"]
    requests = {"far": _tokens(700, V, 1), "edge": _tokens(90, V, 2)}
    ref = _reference(cfg, weights, requests)
    schedules = [replay.whole(requests), replay.tail_one_by_one(requests, tail=70), replay.portions(requests, sizes=(33, 2, 64, 7, 16, 1, 41)),
                 replay.mixed(requests, max_live=2, prompt_frac=0.8, sizes=(50, 3, 24, 2), seed=4)]
    first = None
    for steps in schedules:
        cache = engine.new_cache(replay.trace_peak_tokens(steps, 16) // 16, 16, 2)
        got = replay.run_trace(engine, cache, steps)
        assert _covered(got, requests)
        if dtype == "fp32":
            assert _worst(got, ref) < 2 * F32_TOL       # (scores several times larger carry their rounding into the weights)
        else:
            assert _mean(got, ref) < 6e-2
            first = first or _stacked(got)
            assert np.mean(_errors(got, first)) < 2e-2


def test_one_key_stands_out_far_back_at_the_window_edge_and_among_the_kept(tmp_path):
    """A single layer whose scores are made by hand: the embedding rows of two token ids are made so that a query of id 1
    scores a key of id 2 far above all others. Where that key lies (far back among the kept tokens, on the window's edge,
    one token outside it) then decides the row; the engine follows the plain model in each place, in a prompt and decoded."""
    cfg = zm.config([zm.gated(heads=1, kv_heads=1, dim=16, dims=0, window=24, keep_first=4, scale=1.0, mlp=None)], width=16, vocab=9)
    weights = zm.make_weights(cfg, 31, torch.float32)
    # the query reads the stream's entry 0; a key's entry 0 is the stream's entry 1, its entry 3 the stream's (a value is its key)
    weights["l0.mix.q"], weights["l0.mix.k"] = torch.eye(16), torch.zeros(16, 16)
    weights["l0.mix.k"][0, 1] = 1.0
    weights["l0.mix.k"][3, 3] = 1.0
    weights["l0.norm1"] = torch.zeros(16)
    weights["embed"] = torch.randn(9, 16, generator=torch.Generator().manual_seed(5)) * 0.3
    weights["embed"][1] = 0
    weights["embed"][1, 0] = 6.0
    weights["embed"][2] = 0
    weights["embed"][2, 1] = 5.0
    weights["embed"][2, 3] = 4.0                    # what the row carries when the key is seen
    engine, _ = _engine(tmp_path, cfg, 31, "fp32", weights=weights)
    fill = [3, 4, 5, 6, 7, 8]
    base = [fill[i % 6] for i in range(200)]
    seen = {}
    for where, at in (("kept", 3), ("first outside the kept", 4), ("window edge", 199 - 23), ("one outside the window", 199 - 24),
                      ("page border", 192), ("itself only", None)):
        ids = list(base)
        if at is not None:
            ids[at] = 2
        ids[199] = 1
        requests = {"r": ids}
        ref = _reference(cfg, weights, requests)
        for steps in (replay.whole(requests), replay.tail_one_by_one(requests, tail=3), replay.portions(requests, sizes=(64, 2, 33))):
            got = replay.run_trace(engine, engine.new_cache(14, 16, 1), steps)
            assert _worst(got, ref) < F32_TOL, where
        seen[where] = ref["r"][199]
    moved = lambda a, b: float(np.sqrt(np.mean((seen[a] - seen[b]) ** 2)) / np.sqrt(np.mean(seen[b] ** 2)))
    assert moved("kept", "itself only") > 0.1 and moved("window edge", "itself only") > 0.1 and moved("page border", "itself only") > 0.1
    assert moved("first outside the kept", "itself only") < 1e-6 and moved("one outside the window", "itself only") < 1e-6


def test_long_decoding_through_recorded_steps(tmp_path):
    """300 tokens one by one after a short prompt: windows pass over decoded tokens many times, pages of the sliding
    layers are given back and used again, the kept tokens stay, and the recorded step is replayed."""
    cfg = zm.MIXED
    engine, weights = _engine(tmp_path, cfg, 14, "fp32")
    ids = _tokens(310, cfg["vocab"], 4)
    ref = _reference(cfg, weights, {"r": ids})
    steps = replay.tail_one_by_one({"r": ids}, tail=300)
    got = replay.run_trace(engine, engine.new_cache(20, 16, 2), steps)
    assert _covered(got, {"r": ids}) and _worst(got, ref) < F32_TOL
    assert engine.runner.graph_replays >= 299


def test_long_decoding_in_bfloat16_on_the_matrix_cores(tmp_path):
    cfg = zm.ALIGNED
    engine, weights = _engine(tmp_path, cfg, 18, "bf16")
    ids = _tokens(200, cfg["vocab"], 4)
    whole = _stacked(replay.run_trace(engine, engine.new_cache(16, 16, 1), replay.whole({"r": ids})))
    got = replay.run_trace(engine, engine.new_cache(16, 16, 2), replay.tail_one_by_one({"r": ids}, tail=190))
    assert _mean(got, whole) < BF16_BETWEEN_SCHEDULES / 2 and _most(got, whole) < BF16_BETWEEN_SCHEDULES
    assert engine.runner.graph_replays >= 189


def test_first_tokens_of_a_sequence(tmp_path):
    cfg = zm.MIXED
    engine, weights = _engine(tmp_path, cfg, 15, "fp32")
    requests = {f"n{n}": _tokens(n, cfg["vocab"], 30 + n) for n in range(1, 7)}
    ref = _reference(cfg, weights, requests)
    for steps in (replay.whole(requests), replay.tail_one_by_one(requests, tail=8), replay.mixed(requests, max_live=4, seed=3)):
        got = replay.run_trace(engine, engine.new_cache(8, 16, 4), steps)
        assert _worst(got, ref) < F32_TOL


def test_greedy_generation_through_the_entry_point_and_the_scheduler(tmp_path):
    cfg = zm.MIXED
    engine, weights = _engine(tmp_path, cfg, 16, "fp32")
    prompts = [_tokens(9, cfg["vocab"], 1), _tokens(30, cfg["vocab"], 2), _tokens(1, cfg["vocab"], 3)]
    new = 12
    w = {k: (v.float() if v.is_floating_point() else v) for k, v in weights.items()}

    def plain_greedy(ids):
        ids = list(ids)
        for _ in range(new):
            ids.append(int(plain.forward(cfg, w, ids)[-1].argmax()))
        return ids

    want = [plain_greedy(p) for p in prompts]
    for p, out_want in zip(prompts, want):
        out, finish = engine.generate(p, new)
        assert out == out_want and finish == "length"
    from llmengine import BlockManager, ContinuousBatchScheduler
    sched = ContinuousBatchScheduler(engine, BlockManager(num_blocks=12, block_size=16), max_concurrent=2,
                                     max_prefill_tokens_per_step=16)
    for p in prompts:
        sched.enqueue(p, new)
    sched.run_until_idle()
    assert [r.token_ids for r in sched.results] == want


def test_the_trace_runner_replays_a_model_of_this_design(tmp_path):
    import json
    import os
    import subprocess
    import sys
    cfg = zm.MIXED
    folder, weights = zm.write_model(tmp_path / "model", cfg, 17, torch.float32)
    requests = {"a": _tokens(40, cfg["vocab"], 1), "b": _tokens(21, cfg["vocab"], 2)}
    steps = replay.mixed(requests, max_live=2, seed=5)
    ref = _reference(cfg, weights, requests)
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", str(replay.trace_peak_tokens(steps))],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    done = {rid: 0 for rid in requests}
    for s in steps:
        rows = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, cfg["vocab"])
        r = 0
        for e in s["entries"]:
            for w in e["want"]:
                want = ref[e["id"]][done[e["id"]] + w]
                assert np.sqrt(np.mean((rows[r] - want) ** 2)) / np.sqrt(np.mean(want ** 2)) < F32_TOL
                r += 1
            done[e["id"]] += len(e["tokens"])


def test_the_command_line_generates_with_random_weights_of_this_design(tmp_path):
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfgf = tmp_path / "cfg.json"
    cfgf.write_text(json.dumps(zm.ALIGNED))
    pf = tmp_path / "prompts.txt"
    pf.write_text("1 2 3\n7,8,9,10,11\n")
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "llmengine-cli"), "--random", str(cfgf), "--seed", "3",
                          "--prompt-file", str(pf), "--max-new-tokens", "4", "--temperature", "0.7"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    recs = [json.loads(line) for line in out.stdout.strip().splitlines()]
    assert [len(r["token_ids"]) for r in recs] == [7, 9] and all(r["finish_reason"] == "length" for r in recs)
