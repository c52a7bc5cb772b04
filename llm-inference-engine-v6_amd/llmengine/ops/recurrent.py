"""Python faces of the kernels for residual streams, mixers with a state of fixed size (short
convolutions, the gated diagonal recurrence, the gated delta rule) and attention without a softmax.
As everywhere in ops: operands are checked on the host, then the kernel is launched on the current
stream; nothing computes on the host.

Matrices that are column ranges of a wider buffer are passed as 2-d views whose rows are
contiguous (`stride(1) == 1`); the row stride is their leading dimension.
"""
from __future__ import annotations

import ctypes

import torch

from .lib import KernelError, check, code, declare, entry, ptr, require, stream

_vp, _i, _f, _z = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
_FLOATS = (torch.float32, torch.bfloat16)
MAX_STREAMS = 8
MAX_TAPS = 16
DELTA_MAX_DIM = 256
RGLRU_CHUNK_FROM, RGLRU_CHUNK = 64, 32        # requests that bring more rows than the first are scanned in chunks of the second
GATE_ACTIVATIONS = {"silu": 0, "relu": 1, "gelu_tanh": 2}

declare("llme_streams_spread", [_vp, _i, _z, _vp])
declare("llme_streams_read_norm", [_vp, _i, _i, _i, _vp, _vp, _i, _vp, _i, _vp, _i, _f, _vp])
declare("llme_streams_write", [_vp, _i, _z, _vp, _vp, _vp, _vp])
declare("llme_streams_write_read_norm", [_vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _f, _vp])
declare("llme_gated_act", [_vp, _i, _vp, _i, _i, _i, _i, _i, _vp])
declare("llme_short_conv", [_vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp])
declare("llme_rglru_gates", [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _f, _vp])
declare("llme_rglru_scan", [_vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp])
declare("llme_rglru_scan_chunked", [_vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp])
declare("llme_copy_cols", [_vp, _i, _vp, _i, _i, _i, _vp])
declare("llme_unit_heads", [_vp, _i, _i, _i, _i, _i, _f, _f, _f, _vp])
declare("llme_delta_gates", [_vp, _i, _vp, _i, _vp, _i, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _vp])
declare("llme_delta_rule", [_vp, _i, _i, _i, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _i, _vp, _vp, _vp])
LINEAR_RULE_CHUNK = 64                  # rows of a chunk where the linear rule's long runs of rows are walked side by side
LINEAR_RULE_CHUNK_FROM = 192            # the most rows a request brings from which that is done
LINEAR_RULE_CHUNK_BYTES = 512 << 20     # and the most scratch memory it may take
declare("llme_sigmoid_decay", [_vp, _i, _vp, _i, _vp, _i, _f, _vp, _i, _i, _vp])
declare("llme_gated_head_norm", [_vp, _vp, _vp, _i, _vp, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _f, _f, _vp])
declare("llme_rotate_write", [_vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp])
declare("llme_sigmoid_attention", [_vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _i, _vp])
declare("llme_sigmoid_attention_mfma", [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _vp])
declare("llme_sigmoid_attention_finish", [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _f, _vp])


def _cols(t: torch.Tensor, name: str, dtype, rows: int | None = None, cols: int | None = None) -> int:
    """Checks a 2-d view with contiguous rows; returns its leading dimension."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dim() != 2:
        raise KernelError(f"{name}: expected a 2-d tensor on the GPU")
    allowed = dtype if isinstance(dtype, (tuple, list)) else (dtype,)
    if t.dtype not in allowed:
        raise KernelError(f"{name}: dtype {t.dtype} not in {allowed}")
    if t.shape[1] > 1 and t.stride(1) != 1:
        raise KernelError(f"{name}: rows must be contiguous")
    if (rows is not None and t.shape[0] != rows) or (cols is not None and t.shape[1] != cols):
        raise KernelError(f"{name}: shape {tuple(t.shape)} does not match ({rows}, {cols})")
    ld = t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])
    if ld < t.shape[1]:
        raise KernelError(f"{name}: rows overlap")
    return int(ld)


# --- residual streams ----------------------------------------------------------------
def streams_spread(x: torch.Tensor) -> None:
    """x [S, T, H] (32-bit): every stream becomes a copy of stream 0."""
    require(x, "x", torch.float32, (None, None, None))
    S, T, H = x.shape
    if S > MAX_STREAMS:
        raise KernelError(f"streams: at most {MAX_STREAMS} streams, got {S}")
    check(entry("llme_streams_spread")(ptr(x), S, T * H, stream()), "streams_spread")


def streams_read_norm(x: torch.Tensor, coef: torch.Tensor | None, weight: torch.Tensor | None, eps: float,
                      out: torch.Tensor, rows: torch.Tensor | None = None) -> None:
    """u = sum_s coef[s] x[s] (coef None: the plain sum) at the chosen rows; out = weight * u / sqrt(mean(u^2) + eps),
    or u itself (32-bit) where weight is None."""
    require(x, "x", torch.float32, (None, None, None))
    S, T, H = x.shape
    if S > MAX_STREAMS:
        raise KernelError(f"streams: at most {MAX_STREAMS} streams, got {S}")
    if coef is not None:
        require(coef, "coef", torch.float32, (S,))
    R = T if rows is None else rows.shape[0]
    if rows is not None:
        require(rows, "rows", torch.int32, (R,))
    if weight is not None:
        require(weight, "weight", _FLOATS, (H,))
        require(out, "out", _FLOATS, (R, H))
    else:
        require(out, "out", torch.float32, (R, H))
    check(entry("llme_streams_read_norm")(ptr(x), S, T, H, ptr(coef), ptr(weight), code(weight.dtype) if weight is not None else 0,
                                          ptr(out), code(out.dtype), ptr(rows), R, float(eps), stream()), "streams_read_norm")


def streams_write(x: torch.Tensor, mix: torch.Tensor, coef: torch.Tensor, y: torch.Tensor) -> None:
    """In place, all streams at once from the old ones: x[j] = sum_s mix[s, j] x[s] + coef[j] y."""
    require(x, "x", torch.float32, (None, None, None))
    S, T, H = x.shape
    if S > MAX_STREAMS:
        raise KernelError(f"streams: at most {MAX_STREAMS} streams, got {S}")
    require(mix, "mix", torch.float32, (S, S))
    require(coef, "coef", torch.float32, (S,))
    require(y, "y", torch.float32, (T, H))
    check(entry("llme_streams_write")(ptr(x), S, T * H, ptr(mix), ptr(coef), ptr(y), stream()), "streams_write")


def streams_write_read_norm(x: torch.Tensor, mix: torch.Tensor, coef: torch.Tensor, y: torch.Tensor, next_coef: torch.Tensor,
                            weight: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """streams_write(x, mix, coef, y) and then streams_read_norm(x, next_coef, weight, eps, out), as one kernel where the
    sizes let it (up to 4 streams, rows of a multiple of 4 up to 4,096 values), else as the two."""
    require(x, "x", torch.float32, (None, None, None))
    S, T, H = x.shape
    require(mix, "mix", torch.float32, (S, S))
    require(coef, "coef", torch.float32, (S,))
    require(next_coef, "next_coef", torch.float32, (S,))
    require(y, "y", torch.float32, (T, H))
    require(weight, "weight", _FLOATS, (H,))
    require(out, "out", _FLOATS, (T, H))
    status = entry("llme_streams_write_read_norm")(ptr(x), S, T, H, ptr(mix), ptr(coef), ptr(y), ptr(next_coef), ptr(weight),
                                                   code(weight.dtype), ptr(out), code(out.dtype), float(eps), stream())
    if status == 10002:
        streams_write(x, mix, coef, y)
        streams_read_norm(x, next_coef, weight, eps, out)
        return
    check(status, "streams_write_read_norm")


# --- gated feed-forward activation -------------------------------------------------------
def gated_activation(gu: torch.Tensor, out: torch.Tensor, group: int, activation: str) -> None:
    """out[t, j] = act(gate_j) * up_j from gu [T, 2 FF] laid out in alternating groups; act by name."""
    require(out, "out", _FLOATS, (None, None))
    T, FF = out.shape
    require(gu, "gu", _FLOATS, (T, 2 * FF))
    if activation not in GATE_ACTIVATIONS:
        raise KernelError(f"gated_activation: {activation!r} is none of {sorted(GATE_ACTIVATIONS)}")
    if group <= 0 or FF % group:
        raise KernelError(f"gated_activation: group {group} does not divide the width {FF}")
    if gu.dtype == torch.bfloat16 and out.dtype != torch.bfloat16:
        raise KernelError("gated_activation: bfloat16 input needs bfloat16 output")
    check(entry("llme_gated_act")(ptr(gu), code(gu.dtype), ptr(out), code(out.dtype), T, FF, group,
                                  GATE_ACTIVATIONS[activation], stream()), "gated_activation")


# --- short causal convolution --------------------------------------------------------------
def short_conv(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor | None, tail: torch.Tensor, step,
               out: torch.Tensor, silu: bool, update_tail: bool = True, in_bias: torch.Tensor | None = None) -> None:
    """out[t, c] = act(bias[c] + sum_j taps[c, j] x'[t - (K - 1 - j), c]), x' = x + in_bias, within each request of
    the step; rows before the step come from the request's slot of tail [slots, K - 1, C], which then moves on."""
    T, C = x.shape
    ld_in = _cols(x, "x", torch.float32)
    ld_out = _cols(out, "out", torch.float32, T, C)
    require(taps, "taps", torch.float32, (C, None))
    K = taps.shape[1]
    if not 1 <= K <= MAX_TAPS:
        raise KernelError(f"short_conv: 1 to {MAX_TAPS} taps, got {K}")
    if bias is not None:
        require(bias, "bias", torch.float32, (C,))
    if in_bias is not None:
        require(in_bias, "in_bias", torch.float32, (C,))
    require(tail, "tail", torch.float32, (None, max(K - 1, 0), C))
    if T != step.num_tokens:
        raise KernelError("short_conv: one row per token of the step")
    check(entry("llme_short_conv")(ptr(x), ld_in, ptr(taps), ptr(bias), ptr(in_bias), ptr(tail), ptr(step.seq_idx), ptr(step.q_start),
                                   ptr(step.slots), ptr(out), ld_out, T, step.num_seqs, C, K, 1 if silu else 0,
                                   1 if update_tail else 0, stream()), "short_conv")


# --- gated diagonal recurrence -------------------------------------------------------------
def rglru_gates(u: torch.Tensor, ra: torch.Tensor, ra_bias: torch.Tensor, ri: torch.Tensor, ri_bias: torch.Tensor,
                lam: torch.Tensor, rate: float, decay: torch.Tensor, drive: torch.Tensor) -> None:
    """decay = exp(-rate * sigmoid(Ra u + ba) * softplus(lam)), drive = sqrt(1 - decay^2) * sigmoid(Ri u + bi) * u,
    with Ra, Ri block-diagonal: ra, ri [blocks, bw, bw] ([out, in])."""
    T, width = u.shape
    ld = _cols(u, "u", torch.float32)
    require(ra, "ra", _FLOATS, (None, None, None))
    blocks, bw, _ = ra.shape
    if blocks * bw != width or ra.shape[2] != bw:
        raise KernelError(f"rglru_gates: ra {tuple(ra.shape)} does not tile {width} channels")
    require(ri, "ri", ra.dtype, tuple(ra.shape))
    for t, n in ((ra_bias, "ra_bias"), (ri_bias, "ri_bias"), (lam, "lam")):
        require(t.view(-1), n, torch.float32, (width,))
    require(decay, "decay", torch.float32, (T, width))
    require(drive, "drive", torch.float32, (T, width))
    check(entry("llme_rglru_gates")(ptr(u), ld, ptr(ra), ptr(ra_bias), ptr(ri), ptr(ri_bias), ptr(lam), code(ra.dtype),
                                    ptr(decay), ptr(drive), T, width, blocks, float(rate), stream()), "rglru_gates")


def rglru_scan(decay: torch.Tensor, drive: torch.Tensor, y: torch.Tensor, y_bias: torch.Tensor | None,
               state: torch.Tensor, step, out: torch.Tensor) -> None:
    """s_t = decay_t s_(t-1) + drive_t from each request's slot of state [slots, width];
    out[t] = s_t * gelu_tanh(y[t] + y_bias)."""
    T, width = decay.shape
    require(decay, "decay", torch.float32, (T, width))
    require(drive, "drive", torch.float32, (T, width))
    ld_y = _cols(y, "y", torch.float32, T, width)
    if y_bias is not None:
        require(y_bias, "y_bias", torch.float32, (width,))
    require(state, "state", torch.float32, (None, width))
    ld_out = _cols(out, "out", _FLOATS, T, width)
    if T != step.num_tokens:
        raise KernelError("rglru_scan: one row per token of the step")
    longest = max(step.new_lens) if step.new_lens else T
    if longest > RGLRU_CHUNK_FROM:
        # long runs of rows (prompts): chunks scanned side by side, joined through each chunk's (product, sum)
        chunk = RGLRU_CHUNK
        chunks = (longest + chunk - 1) // chunk
        part = step.buffer("rglru.chunks", (step.num_seqs, chunks, 2, width), torch.float32)
        check(entry("llme_rglru_scan_chunked")(ptr(decay), ptr(drive), ptr(y), ld_y, ptr(y_bias), ptr(state), ptr(step.q_start),
                                               ptr(step.slots), ptr(out), code(out.dtype), ld_out, step.num_seqs, width, chunk,
                                               chunks, ptr(part), stream()), "rglru_scan_chunked")
        return
    check(entry("llme_rglru_scan")(ptr(decay), ptr(drive), ptr(y), ld_y, ptr(y_bias), ptr(state), ptr(step.q_start),
                                   ptr(step.slots), ptr(out), code(out.dtype), ld_out, step.num_seqs, width, stream()),
          "rglru_scan")


# --- gated delta rule ----------------------------------------------------------------------
def copy_cols(src: torch.Tensor, dst: torch.Tensor) -> None:
    """dst [T, n] (contiguous, 32-bit or bfloat16) = src [T, n], a column range of a wider 32-bit buffer."""
    T, n = src.shape
    ld = _cols(src, "src", torch.float32)
    require(dst, "dst", _FLOATS, (T, n))
    check(entry("llme_copy_cols")(ptr(src), ld, ptr(dst), code(dst.dtype), T, n, stream()), "copy_cols")


def unit_heads(x: torch.Tensor, n_a: int, n_b: int, dim: int, scale_a: float, scale_b: float, eps: float) -> None:
    """In place: every head of `dim` entries of x [T, (n_a + n_b) dim] becomes x / sqrt(sum(x^2) + eps), times
    scale_a for the first n_a heads and scale_b for the rest."""
    T = x.shape[0]
    ld = _cols(x, "x", torch.float32, T, (n_a + n_b) * dim)
    check(entry("llme_unit_heads")(ptr(x), ld, T, n_a, n_b, dim, float(scale_a), float(scale_b), float(eps), stream()),
          "unit_heads")


def delta_gates(b_in: torch.Tensor, a_in: torch.Tensor, a2: torch.Tensor | None, A_log: torch.Tensor, dt_bias: torch.Tensor,
                beta: torch.Tensor, decay: torch.Tensor, heads: int, dim: int) -> None:
    """beta = sigmoid(b_in) [T, heads]; decay = exp(-exp(A_log[head]) * softplus(z + dt_bias)) with, per key channel,
    z = a_in a2^T (a2 [heads * dim, rank] given) or z = a_in [T, heads * dim] (a2 None) and decay [T, heads * dim], or per
    head, z = a_in [T, heads] and decay [T, heads]; which of the last two, the shape of `decay` says."""
    T = b_in.shape[0]
    ld_b = _cols(b_in, "b_in", torch.float32, T, heads)
    per_channel = a2 is not None or decay.shape[1] == heads * dim and a_in.shape[1] == heads * dim and dim > 1
    n = heads * dim if per_channel else heads
    rank = 0
    if a2 is not None:
        require(a2, "a2", _FLOATS, (n, None))
        rank = a2.shape[1]
        ld_a = _cols(a_in, "a_in", torch.float32, T, rank)
    else:
        ld_a = _cols(a_in, "a_in", torch.float32, T, n)
    require(A_log, "A_log", torch.float32, (heads,))
    require(dt_bias, "dt_bias", torch.float32, (n,))
    require(beta, "beta", torch.float32, (T, heads))
    require(decay, "decay", torch.float32, (T, n))
    check(entry("llme_delta_gates")(ptr(b_in), ld_b, ptr(a_in), ld_a, ptr(a2), rank, ptr(A_log), ptr(dt_bias),
                                    code(a2.dtype) if a2 is not None else 0, ptr(beta), ptr(decay), T, heads, dim,
                                    1 if per_channel else 0, stream()), "delta_gates")


def sigmoid_decay(z: torch.Tensor, bias: torch.Tensor | None, tau: float, decay: torch.Tensor, a2: torch.Tensor | None = None) -> None:
    """decay [T, n] (32-bit) = sigmoid(z + bias)^(1 / tau), z [T, n] a column range of a 32-bit buffer; with a2 [n, rank],
    z [T, rank] is the first stage of a two-stage map and the logit is z a2^T, summed in 32-bit (bias in a2's type)."""
    T = z.shape[0]
    n = decay.shape[1] if a2 is not None else z.shape[1]
    rank = 0
    if a2 is not None:
        require(a2, "a2", _FLOATS, (n, None))
        rank = a2.shape[1]
        ld = _cols(z, "z", torch.float32, T, rank)
    else:
        ld = _cols(z, "z", torch.float32, T, n)
    if bias is not None:
        require(bias, "bias", a2.dtype if a2 is not None else _FLOATS, (n,))
    require(decay, "decay", torch.float32, (T, n))
    if not tau > 0:
        raise KernelError(f"sigmoid_decay: tau={tau} must be > 0")
    w_dtype = a2.dtype if a2 is not None else bias.dtype if bias is not None else torch.float32
    check(entry("llme_sigmoid_decay")(ptr(z), ld, ptr(a2), rank, ptr(bias), code(w_dtype), float(tau), ptr(decay), T, n, stream()),
          "sigmoid_decay")


def delta_rule(qkv: torch.Tensor, beta: torch.Tensor | None, decay: torch.Tensor, state: torch.Tensor, step, o: torch.Tensor,
               heads: int, kv_heads: int, dim: int, vdim: int, per_channel: bool, q_scale: float = 1.0) -> None:
    """The delta rule over each request's rows, from and into its slot of state [slots, heads, vdim, dim] (M transposed:
    a column's key channels lie together):
    M <- decay * M; w = beta (v - M^T k); M <- M + k w^T; o = q_scale M^T q. beta None: the linear rule, w = v (nothing
    is read back before the write). qkv [T, (2 kv_heads dim + heads vdim)] holds q, k and v side by side; decay is
    [T, heads * dim] (per key channel) or [T, heads]. The linear rule with a decay per channel walks long runs of rows
    (prompts) in chunks side by side: what each chunk adds from an empty memory, the carry from chunk to chunk, then
    every chunk again from the memory in front of it."""
    T = qkv.shape[0]
    ld = _cols(qkv, "qkv", torch.float32, T, 2 * kv_heads * dim + heads * vdim)
    if heads % kv_heads:
        raise KernelError(f"delta_rule: {heads} heads do not divide into {kv_heads} key heads")
    if dim > DELTA_MAX_DIM:
        raise KernelError(f"delta_rule: key size {dim} is beyond the kernel's limit of {DELTA_MAX_DIM}")
    if beta is not None:
        require(beta, "beta", torch.float32, (T, heads))
    require(decay, "decay", torch.float32, (T, None))
    if decay.shape[1] != (heads * dim if per_channel else heads):
        raise KernelError(f"delta_rule: decay has {decay.shape[1]} columns for {heads} heads of {dim}")
    require(state, "state", torch.float32, (None, heads, vdim, dim))
    require(o, "o", torch.float32, (T, heads * vdim))
    if T != step.num_tokens:
        raise KernelError("delta_rule: one row per token of the step")
    chunk, n_chunks, chunk_state, chunk_decay = 0, 0, None, None
    longest = max(step.new_lens) if step.new_lens else T
    if beta is None and per_channel and longest >= LINEAR_RULE_CHUNK_FROM:
        n_chunks = (longest + LINEAR_RULE_CHUNK - 1) // LINEAR_RULE_CHUNK
        places = step.num_seqs * n_chunks
        if places <= 65535 and places * heads * vdim * dim * 4 <= LINEAR_RULE_CHUNK_BYTES:
            chunk = LINEAR_RULE_CHUNK
            chunk_state = step.buffer("linear_rule.chunk_state", (places, heads, vdim, dim), torch.float32)
            chunk_decay = step.buffer("linear_rule.chunk_decay", (places, heads, dim), torch.float32)
    check(entry("llme_delta_rule")(ptr(qkv), ld, 0, kv_heads * dim, 2 * kv_heads * dim, ptr(beta), ptr(decay),
                                   1 if per_channel else 0, ptr(state), ptr(step.q_start), ptr(step.slots), ptr(o),
                                   step.num_seqs, heads, kv_heads, dim, vdim, float(q_scale), chunk, n_chunks if chunk else 0,
                                   ptr(chunk_state), ptr(chunk_decay), stream()), "delta_rule")


def gated_head_norm(o: torch.Tensor, weight: torch.Tensor, gate_in: torch.Tensor, g2: torch.Tensor | None, out: torch.Tensor,
                    heads: int, vdim: int, eps: float, scale: float = 1.0, activation: str = "silu") -> None:
    """out = scale * o / sqrt(mean(o^2) + eps) * weight * gate over every head of o [T, heads * vdim];
    gate = sigmoid(gate_in g2^T) where g2 [heads * vdim, rank] is given, else silu(gate_in) or (activation "sigmoid")
    sigmoid(gate_in) with gate_in [T, heads * vdim]."""
    T = o.shape[0]
    require(o, "o", torch.float32, (T, heads * vdim))
    require(weight, "weight", torch.float32, (vdim,))
    rank = 0
    if g2 is not None:
        require(g2, "g2", _FLOATS, (heads * vdim, None))
        rank = g2.shape[1]
        ld_g = _cols(gate_in, "gate_in", torch.float32, T, rank)
    else:
        ld_g = _cols(gate_in, "gate_in", torch.float32, T, heads * vdim)
    ld_out = _cols(out, "out", _FLOATS, T, heads * vdim)
    check(entry("llme_gated_head_norm")(ptr(o), ptr(weight), ptr(gate_in), ld_g, ptr(g2), rank,
                                        0 if g2 is not None else (2 if activation == "sigmoid" else 1),
                                        code(g2.dtype) if g2 is not None else 0, ptr(out), code(out.dtype), ld_out, T, heads,
                                        vdim, float(eps), float(scale), stream()), "gated_head_norm")


# --- attention without a softmax -------------------------------------------------------------
def rotate_write(qkv: torch.Tensor, inv_freq: torch.Tensor | None, step, block_table: torch.Tensor, q_out: torch.Tensor,
                 k_cache: torch.Tensor, v_cache: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int) -> None:
    """Rotates the q and k heads of qkv [T, heads dim + kv_heads dim + kv_heads vdim] (32-bit) by position * inv_freq
    (pairs (i, i + r / 2), r = 2 len(inv_freq); None: no rotation), writes q to q_out [T, heads dim] and k, v into the
    rows' pages: k_cache [pages, kv_heads, page, dim], v_cache [pages, kv_heads, vdim, page]."""
    T = qkv.shape[0]
    ld = _cols(qkv, "qkv", torch.float32, T, (heads + kv_heads) * dim + kv_heads * vdim)
    rot = 0
    if inv_freq is not None:
        require(inv_freq, "inv_freq", torch.float32, (None,))
        rot = 2 * inv_freq.shape[0]
    if rot > dim:
        raise KernelError(f"rotate_write: {rot} rotated entries in heads of {dim}")
    require(q_out, "q_out", _FLOATS, (T, heads * dim))
    require(k_cache, "k_cache", _FLOATS, (None, kv_heads, None, dim))
    page = k_cache.shape[2]
    require(v_cache, "v_cache", k_cache.dtype, (k_cache.shape[0], kv_heads, vdim, page))
    require(block_table, "block_table", torch.int32, (None, None))
    check(entry("llme_rotate_write")(ptr(qkv), ld, ptr(inv_freq), ptr(step.positions), ptr(step.seq_idx), ptr(block_table),
                                     block_table.shape[1], ptr(q_out), code(q_out.dtype), ptr(k_cache), ptr(v_cache),
                                     code(k_cache.dtype), T, heads, kv_heads, dim, vdim, rot, page, stream()), "rotate_write")


SIGMOID_ATTENTION_LDS = 64 * 1024


def sigmoid_attention_fits(heads: int, dim: int, vdim: int) -> bool:
    return 4 * (heads * dim + heads * heads + heads + 2 * heads * 32) <= SIGMOID_ATTENTION_LDS and heads * vdim <= 256 * 32


def sigmoid_attention_mfma_fits(q: torch.Tensor, heads: int, dim: int, vdim: int, page: int) -> bool:
    """Whether the matrix-core kernel takes these operands (bfloat16, four heads per wavefront, whole matrix tiles)."""
    return (q.dtype == torch.bfloat16 and heads % 4 == 0 and heads <= 32 and dim % 32 == 0 and dim <= 128
            and vdim % 16 == 0 and vdim <= 128 and page % 16 == 0)


SIGMOID_ATTENTION_MFMA_ROWS = 4         # the most rows any request brings must reach this for the matrix-core kernel: a tile of
                                        # 16 rows holding one does the mixing over heads 16 times over on the vector units


def sigmoid_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, mix: torch.Tensor, bias: torch.Tensor,
                      gate: torch.Tensor, step, block_table: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int,
                      dim: int, vdim: int, scale: float, scale_out: float = 1.0, mix_t: torch.Tensor | None = None) -> None:
    """out[t, h] = scale_out * sigmoid(gate[t, h]) * sum_(j <= pos) sigmoid(sum_g mix[h, g] s[g, j] + bias[h]) v_j with
    s[g, j] = scale q_g . k_j over the row's pages. The keys of long requests are cut into runs (one workgroup
    each) whose partial sums are added in a fixed order."""
    T = q.shape[0]
    require(q, "q", _FLOATS, (T, heads * dim))
    require(k_cache, "k_cache", q.dtype, (None, kv_heads, None, dim))
    page = k_cache.shape[2]
    require(v_cache, "v_cache", q.dtype, (k_cache.shape[0], kv_heads, vdim, page))
    require(mix, "mix", torch.float32, (heads, heads))
    require(bias, "bias", torch.float32, (heads,))
    ld_gate = _cols(gate, "gate", torch.float32, T, heads)
    ld_out = _cols(out, "out", _FLOATS, T, heads * vdim)
    require(block_table, "block_table", torch.int32, (None, None))
    if not sigmoid_attention_fits(heads, dim, vdim):
        raise KernelError(f"sigmoid_attention: {heads} heads of {dim} / {vdim} are beyond the kernel's limits")
    # the longest row's keys: from the step's host lists, or what a recorded step is planned for
    if step.plan_len is not None:
        longest = int(step.plan_len)
    else:
        longest = max(c + n for c, n in zip(step.ctx_lens, step.new_lens))
    from .mfma import compute_units
    from .choices import choices_of
    if (mix_t is not None and choices_of(step).fast_attention and max(step.new_lens) >= SIGMOID_ATTENTION_MFMA_ROWS
            and sigmoid_attention_mfma_fits(q, heads, dim, vdim, page)):
        # a request brings several rows (prompts, portions; single tokens of other requests beside them ride along): up to
        # 16 rows of a request to a workgroup, scores and the second product on the matrix cores. The grid follows the
        # step's shape only.
        require(mix_t, "mix_t", torch.float32, (heads, heads))
        tiles = sum((n + 15) // 16 for n in step.new_lens)
        shortest_run = 256 if tiles >= 32 else 64
        runs = max(1, min(64, -(-4 * compute_units() // tiles), (longest + shortest_run - 1) // shortest_run))
        run_len = ((longest + runs - 1) // runs + 31) // 32 * 32
        runs = max(1, (longest + run_len - 1) // run_len)
        partial = step.buffer("sigmoid_attention.partial", (runs, T, heads * vdim), torch.float32)
        check(entry("llme_sigmoid_attention_mfma")(ptr(q), ptr(k_cache), ptr(v_cache), ptr(mix_t), ptr(bias), ptr(step.positions),
                                                   ptr(step.q_start), ptr(block_table), block_table.shape[1], ptr(partial), T,
                                                   step.num_seqs, heads, kv_heads, dim, vdim, page, float(scale), run_len, runs,
                                                   tiles, stream()), "sigmoid_attention_mfma")
        check(entry("llme_sigmoid_attention_finish")(ptr(partial), runs, ptr(gate), ld_gate, ptr(out), code(out.dtype), ld_out, T,
                                                     heads, vdim, float(scale_out), stream()), "sigmoid_attention_finish")
        return
    # steps of single tokens: the kernel for few rows, the keys cut into runs of at least 64 until the chip is full
    runs = max(1, min(64, -(-4 * compute_units() // max(T, 1)), (longest + 63) // 64))
    run_len = (longest + runs - 1) // runs
    run_len = (run_len + 31) // 32 * 32
    runs = max(1, (longest + run_len - 1) // run_len)
    partial = step.buffer("sigmoid_attention.partial", (runs, T, heads * vdim), torch.float32)
    check(entry("llme_sigmoid_attention")(ptr(q), code(q.dtype), ptr(k_cache), ptr(v_cache), code(k_cache.dtype), ptr(mix),
                                          ptr(bias), ptr(step.positions), ptr(step.seq_idx), ptr(block_table),
                                          block_table.shape[1], ptr(partial), T, heads, kv_heads, dim, vdim, page, float(scale),
                                          run_len, runs, stream()), "sigmoid_attention")
    check(entry("llme_sigmoid_attention_finish")(ptr(partial), runs, ptr(gate), ld_gate, ptr(out), code(out.dtype), ld_out, T,
                                                 heads, vdim, float(scale_out), stream()), "sigmoid_attention_finish")
