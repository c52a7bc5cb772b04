"""A plain, slow implementation of the Zetonex design: whole sequences, float64, no cache, no batches,
one function per mechanism. It shares nothing with the engine and is what the engine's results are held
against. Weights come as a dict name -> torch tensor (any float type, integer tables as integers), the
configuration as the dict that config.json holds.

Notation: T tokens, D the residual width, n query heads, g key/value heads, d query/key entries and dv value
entries per head, r rotated entries.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over the root of (the mean of its squares + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w.to(F64)


def norm_centered(x, w, eps):
    """RMS norm whose stored weight is the distance from one."""
    return rms_unit(x, eps) * (1.0 + w.to(F64))


def linear(x, w, b=None):
    y = x @ w.to(F64).T
    return y if b is None else y + b.to(F64)


def silu(z):
    return z * torch.sigmoid(z)


def frequencies(rot: dict) -> torch.Tensor:
    """The angular step of every pair (i, i + dims / 2): base^(-2 i / dims), stretched by wavelength band
    where 'scaling' is given: short waves stay, long waves slow down by the factor, between them a blend."""
    n = int(rot["dims"])
    i = torch.arange(n // 2, dtype=F64)
    f = float(rot["base"]) ** (-2.0 * i / n)
    sc = rot.get("scaling")
    if not sc:
        return f
    factor, low, high, orig = (float(sc[k]) for k in ("factor", "low", "high", "original"))
    wave = 2.0 * math.pi / f
    out = f.clone()
    for j in range(n // 2):
        if wave[j] < orig / high:
            continue
        if wave[j] > orig / low:
            out[j] = f[j] / factor
        else:
            s = (orig / wave[j] - low) / (high - low)
            out[j] = (1.0 - s) * f[j] / factor + s * f[j]
    return out


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, ..., >= dims]: entry i of the first `dims` turns with entry i + dims / 2 by position * f_i."""
    n = int(rot["dims"])
    if n == 0:
        return x.clone()
    ang = positions.to(F64)[:, None] * frequencies(rot)[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [n // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., :n // 2], x[..., n // 2:n]
    out = x.clone()
    out[..., :n // 2] = u * c - v * s
    out[..., n // 2:n] = v * c + u * s
    return out


def visible(T: int, window: int = 0, keep_first: int = 0) -> torch.Tensor:
    """[T, T] True where query i may read key j: j <= i, and, where there is a window, i - j < window or j
    among the first keep_first tokens."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def softmax_heads(q, k, v, scale, mask, softcap=0.0):
    """q [T, n, d], k [T, g, d], v [T, g, dv] -> [T, n, dv]: head h reads key/value head h // (n // g)."""
    T, n, _ = q.shape
    g = k.shape[1]
    out = torch.zeros(T, n, v.shape[2], dtype=F64)
    for h in range(n):
        s = (q[:, h] @ k[:, h // (n // g)].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~mask, -math.inf)
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, h // (n // g)]
    return out


def gated_attention(x, w, m, positions=None):
    """The mixer 'attention': values are the keys before rotation; a window that keeps the first tokens; a
    sigmoid gate on the joined heads. w: the mixer's tensors by local name."""
    T = x.shape[0]
    n, g, d = m["heads"], m["kv_heads"], m["dim"]
    positions = torch.arange(T) if positions is None else positions
    q = linear(x, w["q"]).view(T, n, d)
    k = linear(x, w["k"]).view(T, g, d)
    v = k
    rot = m.get("rot")
    if rot:
        q, k = rotate_halves(q, positions, rot), rotate_halves(k, positions, rot)
    mask = m.get("mask") or {}
    o = softmax_heads(q, k, v, m["scale"], visible(T, mask.get("size", 0), mask.get("keep_first", 0)))
    o = o.reshape(T, n * d) * torch.sigmoid(linear(x, w["g"]))
    return linear(o, w["o"])


def differential_lambda(w, diff):
    return (math.exp(float((w["lq1"].to(F64) * w["lk1"].to(F64)).sum()))
            - math.exp(float((w["lq2"].to(F64) * w["lk2"].to(F64)).sum())) + diff)


def differential_attention(x, w, m, eps, positions=None):
    """The mixer 'attention_2': two softmax maps per head over the same values, the second taken off the
    first lambda times; queries and keys normed per head and map; capped scores; a sliding window."""
    T = x.shape[0]
    n, g, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(T) if positions is None else positions
    q = linear(x, w["q"]).view(T, n, 2, d)
    k = linear(x, w["k"]).view(T, g, 2, d)
    v = linear(x, w["v"]).view(T, g, dv)
    q, k = norm_plain(q, w["q.norm"], eps), norm_plain(k, w["k.norm"], eps)
    rot = m.get("rot")
    if rot:
        q, k = rotate_halves(q, positions, rot), rotate_halves(k, positions, rot)
    mask = visible(T, (m.get("mask") or {}).get("size", 0))
    a1 = softmax_heads(q[:, :, 0], k[:, :, 0], v, m["scale"], mask, m.get("softcap", 0.0))
    a2 = softmax_heads(q[:, :, 1], k[:, :, 1], v, m["scale"], mask, m.get("softcap", 0.0))
    o = a1 - differential_lambda(w, m["diff"]) * a2
    o = rms_unit(o, eps) * (1.0 - m["diff"])
    return linear(o.reshape(T, n * dv), w["o"])


def dense_ff(x, w):
    return linear(silu(linear(x, w["gate"], w["gate.b"])) * linear(x, w["up"], w["up.b"]), w["down"], w["down.b"])


def expert_ff(x, w, e, limit):
    gte = linear(x, w[f"e{e}.gate"]).clamp(max=limit)
    up = linear(x, w[f"e{e}.up"]).clamp(-limit, limit)
    return linear(gte * torch.sigmoid(1.702 * gte) * (up + 1.0), w[f"e{e}.down"])


def table_experts(x, tokens, w, mlp):
    """Every token runs the experts its id names in the table, each weighing 1 / top."""
    top = mlp["router"]["top"]
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e in w["table"][int(tokens[t])].tolist():
            out[t] += expert_ff(x[t:t + 1], w, int(e), mlp["expert"]["limit"])[0] / top
    return out


def sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def layer_order(cfg: dict) -> list[tuple[int, bool]]:
    """(layer, whether the pass input map runs in front of it) in the order the layers run."""
    L = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(L)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(start)]
    for _ in range(times):
        order += [(i, i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, L)]


def forward(cfg: dict, weights: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the residual after every layer run)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = cfg["norm"]["eps"]
    x0 = weights["embed"].to(F64)[tokens]
    x = x0.clone()
    seen = []
    for i, enter in layer_order(cfg):
        layer = cfg["layers"][i]
        if enter:
            x = linear(torch.cat([x, x0], dim=-1), weights["loop.in"])
        h = norm_centered(x, weights[f"l{i}.norm1"], eps)
        mw = sub(weights, f"l{i}.mix.")
        if layer["type"] == "attention":
            y = gated_attention(h, mw, layer["mixer"])
        elif layer["type"] == "attention_2":
            y = differential_attention(h, mw, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp:
            fw = sub(weights, f"l{i}.mlp.")
            y = y + (dense_ff(h, fw) if mlp["kind"] == "dense" else table_experts(h, tokens, fw, mlp))
        x = x + y
        seen.append(x.clone())
    logits = linear(norm_centered(x, weights["final.norm"], eps), weights["head"]) * cfg.get("logit_scale", 1.0)
    return (logits, torch.stack(seen)) if return_layers else logits
