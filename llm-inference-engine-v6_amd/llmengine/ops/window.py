"""Python faces of the kernels for softmax attention with windows that keep the first tokens, several score maps
per value head, capped scores and key and value sizes that differ (csrc/window_attention*.hip), and of the small
kernels around feed-forward layers with biases, clamped gates and experts chosen by a table (csrc/feed_forward.hip).
As everywhere in ops: operands are checked on the host, then the kernel is launched on the current stream."""
from __future__ import annotations

import ctypes

import torch

from .lib import KernelError, check, code, declare, entry, ptr, require, stream

_vp, _i, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_FLOATS = (torch.float32, torch.bfloat16)
WINDOW_ATTENTION_MAX_ENTRIES = 256          # entries of a key or value head that the kernels hold
FINISH_MODES = {"plain": 0, "gate": 1, "difference": 2, "head_gate": 3}
BIAS_ACTIVATIONS = {"silu": 0, "relu": 1, "gelu_tanh": 2, "swish_clamped": 3}

declare("llme_qk_prepare", [_vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _f, _vp, _i, _i, _f, _i, _vp, _vp, _vp, _i, _vp, _i, _vp,
                            _vp, _i, _i, _i, _vp])
declare("llme_window_attention", [_vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _f, _f, _i, _i, _vp,
                                  _vp])
declare("llme_window_attention_finish", [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _i, _f, _f, _f, _vp, _vp, _i, _i, _vp])
declare("llme_gated_bias_act", [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _f, _f, _vp, _vp, _vp])
declare("llme_add_row_bias", [_vp, _vp, _i, _i, _i, _vp])
declare("llme_table_route", [_vp, _vp, _vp, _vp, _i, _i, _vp])
declare("llme_concat_rows", [_vp, _vp, _vp, _i, _i, _i, _vp])


def _columns(p: torch.Tensor, name: str) -> int:
    """A 32-bit matrix whose rows may be wider than what is read of them: returns the row stride."""
    if not isinstance(p, torch.Tensor) or not p.is_cuda or p.dtype != torch.float32 or p.dim() != 2 or p.stride(1) != 1:
        raise KernelError(f"{name}: a 32-bit matrix on the GPU with unit column stride")
    return p.stride(0)


def qk_prepare(p: torch.Tensor, step, block_table: torch.Tensor | None, q_out: torch.Tensor, k_cache: torch.Tensor | None,
               v_cache: torch.Tensor | None, nq: int, k_col: int, v_col: int | None, inv_freq: torch.Tensor | None, rot: int,
               wq: torch.Tensor | None = None, wk: torch.Tensor | None = None, eps: float = 0.0, pairs: str = "halves",
               q_temp: tuple[float, int] | None = None, dk: int | None = None) -> None:
    """Rows p [T, ..] (32-bit: nq query heads of dk entries at column 0, the key heads at k_col, the value heads at
    v_col; v_col None: a value head is the key head as projected) -> q_out [T, nq dk] and the cache entries of the
    rows' tokens: k_cache [pages, nk, page, dk], v_cache [pages, nv, dv, page]. wq, wk [dk]: every query and key
    head is divided by its root mean square (eps inside the root) and multiplied by the weight first. Then the first
    `rot` entries of a query or key head turn by position * inv_freq[i]: entry i with entry i + rot / 2 (pairs
    "halves") or entry 2 i with entry 2 i + 1 ("neighbours"). q_temp (coef, every): the queries of position p times
    1 + coef ln(floor((p + 1) / every) + 1). k_cache None: only the queries are made (the keys and values are another
    layer's; `dk` then says the heads' size)."""
    T = p.shape[0]
    ld = _columns(p, "p")
    if pairs not in ("halves", "neighbours"):
        raise KernelError(f"qk_prepare: pairs {pairs!r} is neither 'halves' nor 'neighbours'")
    if k_cache is not None:
        require(k_cache, "k_cache", _FLOATS, (None, None, None, None))
        _, nk, page, dk = k_cache.shape
        require(v_cache, "v_cache", k_cache.dtype, (k_cache.shape[0], None, None, page))
        nv, dv = v_cache.shape[1], v_cache.shape[2]
        require(block_table, "block_table", torch.int32, (None, None))
        if v_col is None and (nk != nv or dk != dv):
            raise KernelError("qk_prepare: values that are the keys need as many value heads of the same size")
        if (wq is None) != (wk is None):
            raise KernelError("qk_prepare: query and key norm come together")
    else:
        if dk is None or dk <= 0:
            raise KernelError("qk_prepare: queries alone need the heads' size")
        nk = nv = dv = 0
        page, v_col = 1, None
    require(q_out, "q_out", k_cache.dtype if k_cache is not None else _FLOATS, (T, nq * dk))
    need = max(nq * dk, (k_col + nk * dk) if nk else 0, (v_col + nv * dv) if v_col is not None else 0)
    if p.shape[1] < need:
        raise KernelError(f"qk_prepare: rows of {p.shape[1]} columns hold no {need}")
    if rot:
        require(inv_freq, "inv_freq", torch.float32, (rot // 2,))
    if wq is not None:
        require(wq, "wq", _FLOATS, (dk,))
    if wk is not None:
        require(wk, "wk", wq.dtype, (dk,))
    coef, every = (float(q_temp[0]), int(q_temp[1])) if q_temp else (0.0, 0)
    if q_temp and every <= 0:
        raise KernelError("qk_prepare: the queries' temperature steps every > 0 positions")
    check(entry("llme_qk_prepare")(ptr(p), ld, nq, nk, nv, dk, dv, int(k_col), -1 if v_col is None else int(v_col), ptr(wq), ptr(wk),
                                   code(wq.dtype) if wq is not None else 0, float(eps), ptr(inv_freq) if rot else None, int(rot),
                                   1 if pairs == "neighbours" else 0, coef, every,
                                   ptr(step.positions), ptr(step.seq_idx), ptr(block_table) if nk else None,
                                   block_table.shape[1] if nk else 0, ptr(q_out), code(q_out.dtype), ptr(k_cache), ptr(v_cache),
                                   code(q_out.dtype), page, T, stream()), "qk_prepare")


declare("llme_window_attention_mfma", [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _f, _f, _i, _i,
                                       _i, _i, _vp, _vp, _i, _vp, _vp, _i, _f, _vp])
WINDOW_MFMA_FINISHES = True         # a step whose keys are in one run has its rows finished by the attention kernel (False: tests)
WINDOW_MFMA_STAGED = True           # prompts' blocks of keys staged once a workgroup through LDS (False: measurements, tests)
WINDOW_MFMA_MAX_ENTRIES = 128       # entries of a key or value head that the matrix-core kernel holds
WINDOW_MFMA_MAX_RUNS = 32
WINDOW_MFMA_LONG_RUN = 4            # blocks of 32 keys a run from which a step's keys are cut into twice as many runs


def window_mfma_fits(k_cache: torch.Tensor, v_cache: torch.Tensor, choices=None) -> bool:
    """Whether the matrix-core kernel takes this cache: bfloat16, key entries a multiple of 8 and value entries a multiple
    of 16, both up to 128, pages a multiple of 16 tokens."""
    from .choices import DEFAULT
    dk, dv, page = k_cache.shape[3], v_cache.shape[2], k_cache.shape[2]
    return ((choices or DEFAULT).fast_attention and k_cache.dtype == torch.bfloat16 and dk % 8 == 0 and dv % 16 == 0
            and max(dk, dv) <= WINDOW_MFMA_MAX_ENTRIES and page % 16 == 0)


def window_runs(step, rows_per_token: int, key_heads: int, window: int, keep_first: int) -> tuple[int, int]:
    """(the most tokens a request brings, runs to cut a tile's keys into) for the matrix-core kernel: enough wavefronts
    for four a compute unit, a run no shorter than a block of 32 keys. A step of single tokens plans for requests of
    up to step.plan_len keys where that is set (the step may be recorded and replayed for longer requests)."""
    from . import mfma
    decode = step.num_tokens == step.num_seqs
    max_new = 1 if decode else max(step.new_lens)
    if decode and step.plan_len is not None:
        keys = step.plan_len
    else:
        keys = max(c + n for c, n in zip(step.ctx_lens, step.new_lens))
    if window:
        keys = min(keys, window + (16 + rows_per_token - 1) // rows_per_token + min(keep_first, keys))
    tiles = sum((n * rows_per_token + 15) // 16 for n in step.new_lens) * key_heads
    blocks = (keys + 31) // 32 + 1
    runs = max(1, min(WINDOW_MFMA_MAX_RUNS, (4 * mfma.compute_units()) // max(tiles, 1), blocks))
    if decode and blocks > WINDOW_MFMA_LONG_RUN * runs:
        # single tokens over long runs (many keys, no window): twice the wavefronts a compute unit, so that a run is half as long
        runs = max(1, min(WINDOW_MFMA_MAX_RUNS, (8 * mfma.compute_units()) // max(tiles, 1), blocks))
    return max_new, runs


def _fast_window_attention(q, k_cache, v_cache, step, block_table, nq, scale, softcap, window, keep_first, slopes=None, finish=None):
    from .choices import choices_of
    if not window_mfma_fits(k_cache, v_cache, choices_of(step)) or (softcap > 0 and slopes is not None):
        return None
    T = q.shape[0]
    _, nk, page, dk = k_cache.shape
    nv, dv = v_cache.shape[1], v_cache.shape[2]
    max_new, runs = window_runs(step, nq // nk, nk, window, keep_first)
    out = gate = sinks = None
    ld_out = ld_gate = 0
    out_scale = 1.0
    if finish is not None and runs == 1 and nk == nv and finish["mode"] in ("plain", "head_gate") and WINDOW_MFMA_FINISHES:
        o = finish["out"]
        if (o.dtype == torch.bfloat16 and o.stride(1) == 1 and o.stride(0) % 4 == 0 and o.data_ptr() % 8 == 0
                and tuple(o.shape) == (T, nq * dv)):
            # one run of keys: the kernel finishes its rows itself (the sink, the head's gate, the scale)
            out, ld_out, out_scale, sinks = o, o.stride(0), float(finish.get("out_scale", 1.0)), finish.get("sinks")
            if sinks is not None:
                require(sinks, "sinks", torch.float32, (nq,))
            if finish["mode"] == "head_gate":
                gate = finish["gate"]
                ld_gate = _columns(gate, "gate")
                if tuple(gate.shape) != (T, nq):
                    raise KernelError(f"window attention: gate must be [T, {nq}]")
    if out is None:
        part_o = step.buffer("window_attention.part_o", (runs, T, nq, dv), torch.float32)
        part_ml = step.buffer("window_attention.part_ml", (runs, T, nq, 2), torch.float32)
    else:
        part_o = part_ml = None
    check(entry("llme_window_attention_mfma")(ptr(q), ptr(k_cache), ptr(v_cache), ptr(part_o), ptr(part_ml), ptr(step.positions),
                                              ptr(step.q_start), ptr(block_table), block_table.shape[1], T, step.num_seqs, max_new,
                                              nq, nk, nv, dk, dv, page, float(scale), float(softcap), int(window), int(keep_first),
                                              runs, 1 if WINDOW_MFMA_STAGED else 0, ptr(slopes), ptr(out), ld_out, ptr(sinks),
                                              ptr(gate), ld_gate, out_scale, stream()),
          "window_attention_mfma")
    return (part_o, part_ml) if out is None else "finished"


def window_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, step, block_table: torch.Tensor, nq: int,
                     scale: float, softcap: float = 0.0, window: int = 0, keep_first: int = 0,
                     slopes: torch.Tensor | None = None, finish: dict | None = None):
    """Every (token, query head) of the step over the keys of its request that it may see; slopes [heads] (32-bit): the
    score of head h loses slopes[h] times the distance between query and key. finish: what `window_attention_finish`
    would be asked to do with the parts (out, mode, gate, sinks, out_scale); where the matrix-core kernel walks a
    row's keys in one run it does that itself and "finished" is returned instead of the parts. Returns (part_o
    [runs, T, nq, dv], part_ml [runs, T, nq, 2]): per run of keys the unscaled weighted values, the maximum and the
    sum, which `window_attention_finish` joins."""
    T = q.shape[0]
    require(k_cache, "k_cache", _FLOATS, (None, None, None, None))
    _, nk, page, dk = k_cache.shape
    require(v_cache, "v_cache", k_cache.dtype, (k_cache.shape[0], None, None, page))
    nv, dv = v_cache.shape[1], v_cache.shape[2]
    require(q, "q", k_cache.dtype, (T, nq * dk))
    require(block_table, "block_table", torch.int32, (None, None))
    if nk % nv or nq % nk:
        raise KernelError(f"window attention: {nq} query, {nk} key and {nv} value heads do not divide")
    if max(dk, dv) > WINDOW_ATTENTION_MAX_ENTRIES:
        raise KernelError(f"window attention: heads of {dk} and {dv} entries are beyond the kernels' {WINDOW_ATTENTION_MAX_ENTRIES}")
    if slopes is not None:
        require(slopes, "slopes", torch.float32, (nq // (nk // nv),))
    if _fast_window_attention is not None:
        parts = _fast_window_attention(q, k_cache, v_cache, step, block_table, nq, scale, softcap, window, keep_first, slopes, finish)
        if parts is not None:
            return parts
    part_o = step.buffer("window_attention.part_o", (1, T, nq, dv), torch.float32)
    part_ml = step.buffer("window_attention.part_ml", (1, T, nq, 2), torch.float32)
    check(entry("llme_window_attention")(ptr(q), code(q.dtype), ptr(k_cache), ptr(v_cache), code(k_cache.dtype), ptr(part_o),
                                         ptr(part_ml), ptr(step.positions), ptr(step.seq_idx), ptr(block_table),
                                         block_table.shape[1], T, nq, nk, nv, dk, dv, page, float(scale), float(softcap),
                                         int(window), int(keep_first), ptr(slopes), stream()), "window_attention")
    return part_o, part_ml


def window_attention_finish(part_o: torch.Tensor, part_ml: torch.Tensor, out: torch.Tensor, heads: int, mode: str = "plain",
                            gate: torch.Tensor | None = None, lam: float = 0.0, eps: float = 0.0, out_scale: float = 1.0,
                            sinks: torch.Tensor | None = None) -> None:
    """out [T, heads dv] (a view with its own row stride may be given) from the runs' parts. mode "gate": times
    sigmoid(gate), gate [T, heads dv] 32-bit (also a view); "head_gate": the same with one number a head, gate
    [T, heads]; "difference": a head's two maps as a_1 - lam a_2, divided by the root mean square over the head's
    entries (eps inside the root). sinks [heads] 32-bit: the softmax's sum also holds e^(sink). All times out_scale."""
    require(part_o, "part_o", torch.float32, (None, None, None, None))
    runs, T, nq, dv = part_o.shape
    require(part_ml, "part_ml", torch.float32, (runs, T, nq, 2))
    maps = 2 if mode == "difference" else 1
    if mode not in FINISH_MODES or nq != heads * maps:
        raise KernelError(f"window_attention_finish: mode {mode!r} with {nq} query heads for {heads} heads")
    if (not isinstance(out, torch.Tensor) or not out.is_cuda or out.dtype not in _FLOATS or out.dim() != 2 or out.stride(1) != 1
            or tuple(out.shape) != (T, heads * dv)):
        raise KernelError(f"window_attention_finish: out must be [T, {heads * dv}] with unit column stride")
    ld_gate = 0
    if mode in ("gate", "head_gate"):
        ld_gate = _columns(gate, "gate")
        width = heads * dv if mode == "gate" else heads
        if tuple(gate.shape) != (T, width):
            raise KernelError(f"window_attention_finish: gate must be [T, {width}]")
    if sinks is not None:
        require(sinks, "sinks", torch.float32, (heads,))
        if maps != 1:
            raise KernelError("window_attention_finish: a sink goes with one score map a head")
    check(entry("llme_window_attention_finish")(ptr(part_o), ptr(part_ml), runs, T, heads, maps, dv, FINISH_MODES[mode],
                                                ptr(gate) if ld_gate else None, ld_gate, float(lam), float(eps),
                                                float(out_scale), ptr(sinks), ptr(out), code(out.dtype), out.stride(0), stream()),
          "window_attention_finish")


# --- feed-forward layers with biases, clamped gates, experts by table --------------------------------
def gated_bias_act(gu: torch.Tensor, out: torch.Tensor, group: int, activation: str, bias: torch.Tensor | None = None,
                   limit: float = 0.0, alpha: float = 1.0, row_pair: torch.Tensor | None = None,
                   pair_scale: torch.Tensor | None = None) -> None:
    """out [T, FF] = act(gate + b) * (up + b) from gu [T, 2 FF] 32-bit with gate and up columns in alternating groups
    of `group` (bias [2 FF] in the same order). "swish_clamped": g = min(gate, limit), u = clamp(up, -limit, limit),
    out = g sigmoid(alpha g) (u + 1). row_pair [T] int32 with pair_scale (32-bit): row t's gate and up sums are first
    multiplied by pair_scale[row_pair[t]] (0 where row_pair[t] < 0), which is the layer run on that multiple of its input."""
    require(out, "out", _FLOATS, (None, None))
    T, FF = out.shape
    ld = _columns(gu, "gu")
    if gu.shape[0] != T or gu.shape[1] < 2 * FF:
        raise KernelError(f"gated_bias_act: gu {tuple(gu.shape)} does not hold [T, {2 * FF}]")
    if activation not in BIAS_ACTIVATIONS:
        raise KernelError(f"gated_bias_act: {activation!r} is none of {sorted(BIAS_ACTIVATIONS)}")
    if group <= 0 or FF % group:
        raise KernelError(f"gated_bias_act: group {group} does not divide the width {FF}")
    if bias is not None:
        require(bias, "bias", _FLOATS, (2 * FF,))
    if (row_pair is None) != (pair_scale is None):
        raise KernelError("gated_bias_act: a row's pair and the pairs' scales come together")
    if row_pair is not None:
        require(row_pair, "row_pair", torch.int32, (None,))
        require(pair_scale, "pair_scale", torch.float32)
        if row_pair.shape[0] < T:
            raise KernelError(f"gated_bias_act: {row_pair.shape[0]} pairs for {T} rows")
    check(entry("llme_gated_bias_act")(ptr(gu), ld, ptr(bias), code(bias.dtype) if bias is not None else 0, ptr(out), code(out.dtype),
                                       T, FF, group, BIAS_ACTIVATIONS[activation], float(limit), float(alpha), ptr(row_pair),
                                       ptr(pair_scale), stream()),
          "gated_bias_act")


def add_row_bias(x: torch.Tensor, bias: torch.Tensor) -> None:
    """x[t, :] += bias for every row of the 32-bit matrix x."""
    require(x, "x", torch.float32, (None, None))
    require(bias, "bias", _FLOATS, (x.shape[1],))
    check(entry("llme_add_row_bias")(ptr(x), ptr(bias), code(bias.dtype), x.shape[0], x.shape[1], stream()), "add_row_bias")


def table_route(table: torch.Tensor, tokens: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor) -> None:
    """ids[t] = table[tokens[t]] (the experts of a token's id), wts = 1 / top."""
    require(table, "table", torch.int32, (None, None))
    top = table.shape[1]
    T = tokens.shape[0]
    require(tokens, "tokens", torch.int32, (T,))
    require(ids, "ids", torch.int32, (T, top))
    require(wts, "wts", torch.float32, (T, top))
    check(entry("llme_table_route")(ptr(table), ptr(tokens), ptr(ids), ptr(wts), T, top, stream()), "table_route")


def concat_rows(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> None:
    """out [T, 2 H] = [a | b] for 32-bit a, b [T, H], in out's type."""
    require(a, "a", torch.float32, (None, None))
    T, H = a.shape
    require(b, "b", torch.float32, (T, H))
    require(out, "out", _FLOATS, (T, 2 * H))
    check(entry("llme_concat_rows")(ptr(a), ptr(b), ptr(out), code(out.dtype), T, H, stream()), "concat_rows")
