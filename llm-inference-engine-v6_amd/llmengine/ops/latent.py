"""Python faces of the kernels for sandwich norms, latent attention and mixtures of experts. As everywhere
in ops: operands are checked on the host, then the kernel is launched on the current stream; nothing
computes on the host."""
from __future__ import annotations

import ctypes

import torch

from .lib import KernelError, check, code, declare, entry, ptr, require, stream

_vp, _i, _f, _z, _l = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t, ctypes.c_long
_FLOATS = (torch.float32, torch.bfloat16)
LATENT_MAX_ROW, LATENT_MAX_RANK = 1024, 512         # the plain attention kernel's limits (cached row, latent)
MOE_MAX_EXPERTS = 1024
MOE_TILE = 16

declare("llme_norm_add", [_vp, _vp, _i, _vp, _vp, _i, _vp, _i, _i, _i, _f, _vp])
declare("llme_scale_f32", [_vp, _z, _f, _vp])
declare("llme_latent_prepare", [_vp, _i, _i, _i, _i, _i, _vp, _vp, _i, _vp, _f, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _f, _vp])
declare("llme_latent_q_rotate", [_vp, _i, _vp, _f, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp])
declare("llme_head_gemm", [_vp, _i, _l, _l, _vp, _i, _vp, _i, _l, _l, _i, _i, _i, _i, _vp])
declare("llme_latent_attention", [_vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _vp])
declare("llme_moe_route", [_vp, _i, _i, _i, _f, _i, _i, _vp, _vp, _vp])
declare("llme_moe_plan", [_vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp])
declare("llme_moe_gemm", [_vp, _i, _vp, _i, _i, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp])
declare("llme_moe_combine", [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp])


# --- sandwich norm ---------------------------------------------------------------------
def norm_add(y: torch.Tensor, w_post: torch.Tensor, h: torch.Tensor, eps: float, w_next: torch.Tensor | None = None,
             x_out: torch.Tensor | None = None) -> None:
    """h += w_post * y / rms(y); with w_next also x_out = w_next * h / rms(h) of the updated rows; with x_out and no
    w_next, x_out = the updated rows as they are, in x_out's type. y, h [T, H] 32-bit; the weights multiply as they are."""
    require(y, "y", torch.float32, (None, None))
    T, H = y.shape
    require(h, "h", torch.float32, (T, H))
    require(w_post, "w_post", _FLOATS, (H,))
    if w_next is not None:
        require(w_next, "w_next", w_post.dtype, (H,))
    if w_next is not None or x_out is not None:
        require(x_out, "x_out", _FLOATS, (T, H))
    check(entry("llme_norm_add")(ptr(y), ptr(w_post), code(w_post.dtype), ptr(h), ptr(w_next),
                                 code(w_next.dtype) if w_next is not None else 0, ptr(x_out),
                                 code(x_out.dtype) if x_out is not None else 0, T, H, float(eps), stream()), "norm_add")


def scale_(x: torch.Tensor, s: float) -> None:
    """x *= s, in place (32-bit)."""
    require(x, "x", torch.float32)
    check(entry("llme_scale_f32")(ptr(x), x.numel(), float(s), stream()), "scale")


def zero_(t: torch.Tensor) -> None:
    """Fills a contiguous buffer with zeros (a fill kernel, never a memset: the launch may be recorded)."""
    from .kernels import clear
    if t.is_contiguous() and (t.numel() * t.element_size()) % 16 == 0 and t.data_ptr() % 16 == 0:
        clear(t.view(-1).view(torch.float32))
    else:
        t.zero_()


# --- latent attention ------------------------------------------------------------------
def latent_prepare(p: torch.Tensor, q_rank: int, kv_rank: int, rot: int, rot_dims: int, wq: torch.Tensor, wc: torch.Tensor | None,
                   freq: torch.Tensor | None, mag: float, step, block_table: torch.Tensor | None, cq: torch.Tensor,
                   cache: torch.Tensor | None, eps: float) -> None:
    """p [T, >= q_rank + kv_rank + rot] 32-bit (the down maps' outputs side by side) -> cq [T, q_rank], the
    RMS-normed query latent, and the cache rows [normed latent | shared key part, its first rot_dims entries
    rotated] at the tokens' places. kv_rank = 0: queries only (a layer that reads another layer's rows)."""
    require(p, "p", torch.float32, (None, None))
    T, ld = p.shape
    if ld < q_rank + kv_rank + rot:
        raise KernelError(f"latent_prepare: rows of {ld} hold no {q_rank} + {kv_rank} + {rot} columns")
    require(wq, "wq", _FLOATS, (q_rank,))
    require(cq, "cq", _FLOATS, (T, q_rank))
    page = 0
    if kv_rank:
        require(wc, "wc", wq.dtype, (kv_rank,))
        require(cache, "cache", cq.dtype, (None, None, kv_rank + rot))
        require(block_table, "block_table", torch.int32, (None, None))
        page = cache.shape[1]
        if rot_dims:
            require(freq, "freq", torch.float32, (rot_dims // 2,))
    check(entry("llme_latent_prepare")(
        ptr(p), ld, q_rank, kv_rank, rot if kv_rank else 0, rot_dims if kv_rank else 0, ptr(wq), ptr(wc) if kv_rank else None, code(wq.dtype),
        ptr(freq) if (kv_rank and rot_dims) else None, float(mag), ptr(step.positions), ptr(step.seq_idx),
        ptr(block_table) if kv_rank else None, block_table.shape[1] if kv_rank else 0, ptr(cq),
        ptr(cache) if kv_rank else None, code(cq.dtype), page, T, float(eps), stream()), "latent_prepare")


def latent_q_rotate(q: torch.Tensor, freq: torch.Tensor | None, mag: float, positions: torch.Tensor, qp: torch.Tensor,
                    heads: int, dim: int, rot: int, rot_dims: int, kv_rank: int) -> None:
    """The last `rot` entries of every head of q [T, heads (dim + rot)], the first rot_dims of them rotated,
    into the last `rot` entries of every head of qp [T, heads (kv_rank + rot)]."""
    T = q.shape[0]
    require(q, "q", _FLOATS, (T, heads * (dim + rot)))
    require(qp, "qp", q.dtype, (T, heads * (kv_rank + rot)))
    if rot_dims:
        require(freq, "freq", torch.float32, (rot_dims // 2,))
    require(positions, "positions", torch.int32, (T,))
    check(entry("llme_latent_q_rotate")(ptr(q), code(q.dtype), ptr(freq) if rot_dims else None, float(mag), ptr(positions),
                                        ptr(qp), T, heads, dim, rot, rot_dims, kv_rank, stream()), "latent_q_rotate")


_fast_head_gemm = None          # set by ops/latent_mfma.py


def head_gemm(a: torch.Tensor, a_cols: int, w: torch.Tensor, out: torch.Tensor, out_cols: int, heads: int,
              choices=None) -> None:
    """out[t, h, :N] = w[h] a[t, h, :K] for w [heads, N, K]; a [T, heads * a_cols] and out [T, heads * out_cols]
    hold a head's K inputs and N outputs at the start of its a_cols / out_cols columns."""
    require(w, "w", _FLOATS, (heads, None, None))
    _, N, K = w.shape
    T = a.shape[0]
    require(a, "a", _FLOATS, (T, heads * a_cols))
    require(out, "out", a.dtype, (T, heads * out_cols))
    if K > a_cols or N > out_cols:
        raise KernelError(f"head_gemm: {K} inputs and {N} outputs do not fit heads of {a_cols} and {out_cols} columns")
    if _fast_head_gemm is not None and _fast_head_gemm(a, a_cols, w, out, out_cols, heads, choices):
        return
    check(entry("llme_head_gemm")(ptr(a), code(a.dtype), heads * a_cols, a_cols, ptr(w), code(w.dtype), ptr(out),
                                  code(out.dtype), heads * out_cols, out_cols, T, heads, N, K, stream()), "head_gemm")


def latent_attention_fits(kv_rank: int, rot: int) -> bool:
    return kv_rank <= LATENT_MAX_RANK and kv_rank + rot <= LATENT_MAX_ROW


_fast_latent_attention = None   # set by ops/latent_mfma.py


def latent_attention(qp: torch.Tensor, cache: torch.Tensor, out: torch.Tensor, step, block_table: torch.Tensor,
                     heads: int, kv_rank: int, scale: float, window: int = 0) -> None:
    """out[t, h] = sum_j softmax_j(scale qp[t, h] . row_j) row_j[:kv_rank] over the rows of the token's request
    that it may see (all up to its own; with a window the last `window` of them)."""
    T = qp.shape[0]
    require(cache, "cache", _FLOATS, (None, None, None))
    D = cache.shape[2]
    require(qp, "qp", cache.dtype, (T, heads * D))
    require(out, "out", qp.dtype, (T, heads * kv_rank))
    require(block_table, "block_table", torch.int32, (None, None))
    if not latent_attention_fits(kv_rank, D - kv_rank):
        raise KernelError(f"latent attention: rows of {D} with a latent of {kv_rank} are beyond the kernel's limits")
    if _fast_latent_attention is not None and _fast_latent_attention(qp, cache, out, step, block_table, heads, kv_rank,
                                                                     scale, window):
        return
    check(entry("llme_latent_attention")(ptr(qp), code(qp.dtype), ptr(cache), code(cache.dtype), ptr(out),
                                         ptr(step.positions), ptr(step.seq_idx), ptr(block_table), block_table.shape[1],
                                         T, heads, kv_rank, D, cache.shape[1], float(scale), int(window), stream()),
          "latent_attention")


# --- latent attention on the matrix cores ------------------------------------------------
declare("llme_latent_attention_mfma", [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i,
                                       _l, _l, _l, _l, _vp])
declare("llme_latent_q_split", [_vp, _vp, _f, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp])
declare("llme_heads_to_rows", [_vp, _vp, _i, _i, _i, _vp])
LATENT_MFMA_MAX_ROW, LATENT_MFMA_MAX_RANK = 576, 512


def latent_mfma_fits(cache: torch.Tensor, kv_rank: int, rot: int, choices=None) -> bool:
    """Whether the matrix-core kernel takes these rows: bfloat16, a latent that is a multiple of 16, rows a multiple of 32,
    pages a multiple of 16."""
    from .choices import DEFAULT
    D = kv_rank + rot
    return ((choices or DEFAULT).fast_attention and cache.dtype == torch.bfloat16 and kv_rank % 16 == 0 and D % 32 == 0 and rot % 8 == 0
            and cache.shape[1] % 16 == 0 and D <= LATENT_MFMA_MAX_ROW and kv_rank <= LATENT_MFMA_MAX_RANK)


def latent_splits(step, heads: int, window: int) -> tuple[int, int]:
    """(the most tokens a request brings, runs to cut the keys into) for the matrix-core kernel: enough workgroups for two a
    compute unit, runs of 128 keys at least (runs of 64 were measured no faster). A step of single tokens plans for requests of up to step.plan_len keys where that
    is set (the step may be recorded and replayed for longer requests)."""
    from . import mfma
    decode = step.num_tokens == step.num_seqs
    max_new = 1 if decode else max(step.new_lens)
    if decode and step.plan_len is not None:
        keys = step.plan_len
    else:
        keys = max(c + n for c, n in zip(step.ctx_lens, step.new_lens))
    if window:
        keys = min(keys, window + max_new)
    groups = (max_new * heads + 63) // 64 * step.num_seqs
    return max_new, max(1, min(32, (2 * mfma.compute_units()) // groups, (keys + 127) // 128))


def latent_attention_mfma(qa: torch.Tensor, qr: torch.Tensor | None, cache: torch.Tensor, out: torch.Tensor, step,
                          block_table: torch.Tensor, heads: int, kv_rank: int, scale: float, window: int, head_major: bool) -> None:
    """The matrix-core kernel. qa [T, heads, kv_rank] and qr [T, heads, rot] (head_major: [heads, T, ..]); out as qa."""
    T = step.num_tokens
    D = cache.shape[2]
    rot = D - kv_rank
    require(cache, "cache", torch.bfloat16, (None, None, D))
    require(qa, "qa", torch.bfloat16)
    require(out, "out", torch.bfloat16)
    if qa.numel() != T * heads * kv_rank or out.numel() != qa.numel() or (rot and (qr is None or qr.numel() != T * heads * rot)):
        raise KernelError("latent attention: the queries do not fit the step")
    if rot:
        require(qr, "qr", torch.bfloat16)
    max_new, nsplit = latent_splits(step, heads, window)
    ws_o = ws_ml = None
    if nsplit > 1:
        ws_o = step.buffer("latent.split_sums", (nsplit, heads * T, kv_rank), torch.float32)
        ws_ml = step.buffer("latent.split_stats", (nsplit, heads * T, 2), torch.float32)
    ts, hs = (1, T) if head_major else (heads, 1)
    check(entry("llme_latent_attention_mfma")(
        ptr(qa), ptr(qr) if rot else None, ptr(cache), ptr(out), ptr(ws_o), ptr(ws_ml), ptr(step.positions), ptr(step.q_start),
        ptr(block_table), block_table.shape[1], T, step.num_seqs, max_new, heads, kv_rank, rot, cache.shape[1], float(scale),
        int(window), nsplit, ts, hs, ts, hs, stream()), "latent_attention_mfma")


def latent_q_split(q: torch.Tensor, freq: torch.Tensor | None, mag: float, positions: torch.Tensor, qn: torch.Tensor,
                   qr: torch.Tensor | None, heads: int, dim: int, rot: int, rot_dims: int) -> None:
    """q [T, heads (dim + rot)] -> qn [heads, T, dim], the unrotated entries, and qr [heads, T, rot], the rotated ones."""
    T = q.shape[0]
    require(q, "q", torch.bfloat16, (T, heads * (dim + rot)))
    require(qn, "qn", torch.bfloat16, (heads, T, dim))
    if rot:
        require(qr, "qr", torch.bfloat16, (heads, T, rot))
    check(entry("llme_latent_q_split")(ptr(q), ptr(freq) if rot_dims else None, float(mag), ptr(positions), ptr(qn),
                                       ptr(qr) if rot else None, T, heads, dim, rot, rot_dims, stream()), "latent_q_split")


def heads_to_rows(o: torch.Tensor, out: torch.Tensor) -> None:
    """o [heads, T, c] -> out [T, heads * c]."""
    require(o, "o", torch.bfloat16, (None, None, None))
    n, T, c = o.shape
    require(out, "out", torch.bfloat16, (T, n * c))
    check(entry("llme_heads_to_rows")(ptr(o), ptr(out), T, n, c, stream()), "heads_to_rows")


# --- products in groups on the matrix cores -------------------------------------------------
declare("llme_gemm_bf16_grouped", [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _i, _l, _i, _i, _vp])


def _grouped_fits(a: torch.Tensor, w: torch.Tensor, choices) -> bool:
    from .choices import DEFAULT
    return ((choices or DEFAULT).fast_gemm and a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and w.shape[-1] % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and a.numel() * 2 < (1 << 32) - 65536)


def heads_gemm_fits(a: torch.Tensor, w: torch.Tensor, choices=None) -> bool:
    return _grouped_fits(a, w, choices)


def heads_gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out[h] = a[h] w[h]^T for a [heads, T, K], w [heads, N, K], out [heads, T, N], all bfloat16: the matrix-core tile
    kernel with a matrix per group of row tiles."""
    require(a, "a", torch.bfloat16, (None, None, None))
    n, T, K = a.shape
    require(w, "w", torch.bfloat16, (n, None, K))
    N = w.shape[1]
    require(out, "out", torch.bfloat16, (n, T, N))
    tile = 128 if T >= 512 else 64
    check(entry("llme_gemm_bf16_grouped")(ptr(a), ptr(w), ptr(out), code(out.dtype), 0, N, K, tile, 0, None, None, None, 1,
                                          n * T, n, T, stream()), "heads_gemm")


# --- mixture of experts ----------------------------------------------------------------
MOE_FAST_TILES = (64, 128)


def moe_tile(x: torch.Tensor, w: torch.Tensor, pairs: int, experts: int, group: int, choices=None) -> int:
    """Rows of a tile for a step's grouped products: 16 for the plain-precision kernel; 64 or 128 on the matrix cores
    (bfloat16, gate and up rows interleaved in groups of 16)."""
    if not _grouped_fits(x, w, choices) or group != 16:
        return MOE_TILE
    return 128 if pairs >= 128 * experts else 64


def moe_capacity(pairs: int, experts: int, tile: int = MOE_TILE) -> int:
    """Places for `pairs` (token, expert) pairs when every expert's run is padded to whole tiles."""
    return (pairs + experts * (tile - 1) + tile - 1) // tile * tile


def moe_route(logits: torch.Tensor, top: int, scale: float, renormalize: bool, ids: torch.Tensor, wts: torch.Tensor,
              scoring: str = "softmax") -> None:
    """ids, wts [T, top]: every row's `top` experts with the largest scores, softmax over the row or ("sigmoid") a
    sigmoid of each logit, and their weights score * scale (over the chosen scores' sum first where `renormalize`)."""
    if scoring not in ("softmax", "sigmoid"):
        raise KernelError(f"moe_route: scoring {scoring!r} is neither 'softmax' nor 'sigmoid'")
    require(logits, "logits", torch.float32, (None, None))
    T, E = logits.shape
    require(ids, "ids", torch.int32, (T, top))
    require(wts, "wts", torch.float32, (T, top))
    check(entry("llme_moe_route")(ptr(logits), T, E, top, float(scale), 1 if renormalize else 0, 1 if scoring == "sigmoid" else 0,
                                  ptr(ids), ptr(wts), stream()),
          "moe_route")


def moe_plan(ids: torch.Tensor, experts: int, tile: int, place_pair: torch.Tensor, pair_place: torch.Tensor,
             tile_expert: torch.Tensor, n_tiles: torch.Tensor) -> None:
    require(ids, "ids", torch.int32, (None, None))
    pairs = ids.numel()
    cap = moe_capacity(pairs, experts, tile)
    require(place_pair, "place_pair", torch.int32, (cap,))
    require(pair_place, "pair_place", torch.int32, (pairs,))
    require(tile_expert, "tile_expert", torch.int32, (cap // tile,))
    require(n_tiles, "n_tiles", torch.int32, (1,))
    check(entry("llme_moe_plan")(ptr(ids), pairs, experts, tile, cap, ptr(place_pair), ptr(pair_place), ptr(tile_expert),
                                 ptr(n_tiles), stream()), "moe_plan")


def moe_gemm(a: torch.Tensor, w: torch.Tensor, gated: bool, group: int, out: torch.Tensor, place_pair: torch.Tensor,
             tile_expert: torch.Tensor, n_tiles: torch.Tensor, tile: int, gather_div: int, activation: str = "silu",
             choices=None) -> None:
    """Per place: out[place] = w[expert] a[row]; gated: act(gate a) * (up a), w [experts, 2 N, K] holding gate and up rows in
    alternating groups of `group`. row = pair // gather_div, or the place itself where gather_div is 0."""
    from .recurrent import GATE_ACTIVATIONS
    require(w, "w", _FLOATS, (None, None, None))
    E, rows_w, K = w.shape
    N = rows_w // 2 if gated else rows_w
    require(a, "a", _FLOATS, (None, K))
    cap = place_pair.shape[0]
    require(out, "out", _FLOATS, (cap, N))
    require(tile_expert, "tile_expert", torch.int32, (cap // tile,))
    if gather_div == 0 and a.shape[0] != cap:
        raise KernelError("moe_gemm: rows by place need one row per place")
    if (tile in MOE_FAST_TILES and _grouped_fits(a, w, choices) and (not gated or (group == 16 and activation == "silu"
                                                                                  and out.dtype == torch.bfloat16))):
        check(entry("llme_gemm_bf16_grouped")(ptr(a), ptr(w), ptr(out), code(out.dtype), 1 if gated else 0, rows_w, K, tile,
                                              cap // tile, ptr(tile_expert), ptr(n_tiles), ptr(place_pair) if gather_div else None,
                                              max(gather_div, 1), a.shape[0], E, 0, stream()), "moe_gemm")
        return
    check(entry("llme_moe_gemm")(ptr(a), code(a.dtype), ptr(w), 1 if gated else 0, code(w.dtype), ptr(out), code(out.dtype),
                                 ptr(place_pair), ptr(tile_expert), ptr(n_tiles), tile, cap // tile, int(gather_div), N, K,
                                 int(group), GATE_ACTIVATIONS[activation], stream()), "moe_gemm")


declare("llme_gemm_bf16_grouped_gated_extra", [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _i, ctypes.c_long, _i, _f, _f, _vp, _vp])


def moe_gemm_clamped(a: torch.Tensor, w: torch.Tensor, group: int, out: torch.Tensor, place_pair: torch.Tensor,
                     tile_expert: torch.Tensor, n_tiles: torch.Tensor, tile: int, gather_div: int, limit: float, alpha: float,
                     choices=None, pair_scale: torch.Tensor | None = None) -> bool:
    """The experts' gate/up product with the clamped swish in the tile kernel's epilogue, where that fits (returns False
    where not): per place, g = min(gate a, limit), u = clamp(up a, -limit, limit), out[place] = g sigmoid(alpha g) (u + 1);
    w [experts, 2 N, K] with gate and up rows in alternating groups of 16. pair_scale [pairs] (32-bit): a place's two sums
    are first multiplied by its pair's entry (an expert that runs on its weight times the input); with limit 0 the
    activation is then SiLU."""
    require(w, "w", _FLOATS, (None, None, None))
    E, rows_w, K = w.shape
    if not (tile in MOE_FAST_TILES and _grouped_fits(a, w, choices) and group == 16 and out.dtype == torch.bfloat16
            and rows_w % 32 == 0 and gather_div > 0 and (limit > 0 or (limit == 0 and pair_scale is not None))):
        return False
    if pair_scale is not None:
        require(pair_scale, "pair_scale", torch.float32, (None,))
    require(a, "a", torch.bfloat16, (None, K))
    cap = place_pair.shape[0]
    require(out, "out", torch.bfloat16, (cap, rows_w // 2))
    require(tile_expert, "tile_expert", torch.int32, (cap // tile,))
    check(entry("llme_gemm_bf16_grouped_gated_extra")(ptr(a), ptr(w), ptr(out), rows_w, K, tile, cap // tile, ptr(tile_expert),
                                                      ptr(n_tiles), ptr(place_pair), int(gather_div), a.shape[0], E, float(limit),
                                                      float(alpha), ptr(pair_scale), stream()), "moe_gemm_clamped")
    return True


def moe_combine(y: torch.Tensor, pair_place: torch.Tensor, wts: torch.Tensor | None, out: torch.Tensor, accumulate: bool,
                top: int | None = None) -> None:
    """out[t] (+)= sum_k wts[t, k] y[place of pair (t, k)]; wts None: every one of a token's `top` results counts once."""
    require(out, "out", torch.float32, (None, None))
    T, H = out.shape
    if wts is not None:
        require(wts, "wts", torch.float32, (T, None))
        top = wts.shape[1]
    elif top is None or top <= 0:
        raise KernelError("moe_combine: without weights the number of results a token has must be given")
    require(y, "y", torch.float32, (None, H))
    require(pair_place, "pair_place", torch.int32, (T * top,))
    check(entry("llme_moe_combine")(ptr(y), ptr(pair_place), ptr(wts), ptr(out), T, top, H, 1 if accumulate else 0, stream()),
          "moe_combine")
