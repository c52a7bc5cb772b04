"""A plain, slow implementation of the Zapolorn design: whole sequences, float64, no cache, no batches,
one function per mechanism. It shares nothing with the engine and is what the engine's results are held
against. Weights come as a dict name -> torch tensor (any float type), the configuration as the dict that
config.json holds.

Notation: T tokens, D the residual width, n query heads, g key/value heads, d query/key entries and dv value
entries per head, r rotated entries; i is the position of a query and j that of a key.

The layer: x <- x + N1(mixer(x)); x <- x + N2(ff(x)), the sublayers reading x itself and the norms standing
behind them.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over the root of (the mean of its squares + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms_unit(x, eps) * w.to(F64)


def linear(x, w, b=None):
    y = x @ w.to(F64).T
    return y if b is None else y + b.to(F64)


def silu(z):
    return z * torch.sigmoid(z)


# ---- positions ---------------------------------------------------------------------------------------
def pair_frequencies(rot: dict) -> torch.Tensor:
    """The angular step of pair c = (2c, 2c + 1): base^(-2c / dims), every one divided by the scaling factor."""
    r = int(rot["dims"])
    c = torch.arange(r // 2, dtype=F64)
    f = float(rot["base"]) ** (-2.0 * c / r)
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    return f / factor


def rotate_neighbours(x: torch.Tensor, positions: torch.Tensor, rot: dict | None) -> torch.Tensor:
    """x [T, heads, >= dims]: entries 2c and 2c + 1 of the first `dims` turn together by position * f_c; the
    entries behind them pass."""
    if not rot or not int(rot["dims"]):
        return x.clone()
    r = int(rot["dims"])
    ang = positions.to(F64)[:, None] * pair_frequencies(rot)[None, :]          # [T, r / 2]
    cs, sn = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0:r:2], x[..., 1:r:2]
    out = x.clone()
    out[..., 0:r:2] = a * cs - b * sn
    out[..., 1:r:2] = b * cs + a * sn
    return out


def query_temperature(positions: torch.Tensor, qt: dict | None) -> torch.Tensor:
    """[T]: 1 + coef ln(floor((i + 1) / every) + 1), the factor on the queries of position i."""
    if not qt:
        return torch.ones(len(positions), dtype=F64)
    steps = torch.div(positions + 1, int(qt["every"]), rounding_mode="floor").to(F64)
    return 1.0 + float(qt["coef"]) * torch.log(steps + 1.0)


def head_slopes(n: int) -> torch.Tensor:
    """[n]: head h (from 0) loses 2^(-8 (h + 1) / n) per token of distance."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / n) for h in range(n)], dtype=F64)


def visible(T: int, window: int = 0) -> torch.Tensor:
    """[T, T] True where query i may read key j: j <= i and, under a window, i - j < window."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok = ok & (i - j < window)
    return ok


# ---- softmax attention -------------------------------------------------------------------------------
def attend(q, k, v, scale, mask, slopes=None, sinks=None):
    """q [T, n, d], k [T, g, d], v [T, g, dv] -> [T, n, dv]; head h reads key/value head h // (n // g). A score is
    scale q.k - slope_h (i - j); with `sinks` [n] the denominator also holds e^(sink_h), which has no value."""
    T, n, _ = q.shape
    g = k.shape[1]
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(F64)
    out = torch.zeros(T, n, v.shape[2], dtype=F64)
    for h in range(n):
        kv = h // (n // g)
        s = (q[:, h] @ k[:, kv].T) * scale
        if slopes is not None:
            s = s - slopes[h] * dist
        s = s.masked_fill(~mask, -math.inf)
        top = s.max(dim=-1, keepdim=True).values
        if sinks is not None:
            top = torch.maximum(top, sinks[h].to(F64).expand_as(top))
        e = torch.exp(s - top)
        den = e.sum(-1, keepdim=True)
        if sinks is not None:
            den = den + torch.exp(sinks[h].to(F64) - top)
        out[:, h] = (e / den) @ v[:, kv]
    return out


def keys_values(x, w, m, eps, positions):
    """What a layer of type 'attention' caches: keys after norm and rotation [T, g, d], values [T, g, dv]."""
    T = x.shape[0]
    g, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = norm(linear(x, w["k"]).view(T, g, d), w["k.norm"], eps)
    return rotate_neighbours(k, positions, m.get("rot")), linear(x, w["v"]).view(T, g, dv)


def window_attention(x, w, m, eps, positions=None, kv=None):
    """The mixer 'attention': normed and rotated queries and keys, a sliding window, a sink in the softmax, a
    sigmoid gate per head on the heads' results. kv: keys and values of the layer that `kv_from` names."""
    T = x.shape[0]
    n, d, dv = m["heads"], m["dim"], m["vdim"]
    positions = torch.arange(T) if positions is None else positions
    q = norm(linear(x, w["q"]).view(T, n, d), w["q.norm"], eps)
    q = rotate_neighbours(q, positions, m.get("rot"))
    k, v = kv if kv is not None else keys_values(x, w, m, eps, positions)
    o = attend(q, k, v, m["scale"], visible(T, (m.get("mask") or {}).get("size", 0)), sinks=w["sink"])
    o = o * torch.sigmoid(linear(x, w["g"]))[:, :, None]
    return linear(o.reshape(T, n * dv), w["o"])


def biased_attention(x, w, m, eps, positions=None):
    """The left side of the mixer 'parallel': no rotation; normed queries and keys, queries times a temperature
    that grows with the position, scores that lose slope_h per token of distance, every earlier token visible."""
    T = x.shape[0]
    n, g, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(T) if positions is None else positions
    q = norm(linear(x, w["q"]).view(T, n, d), w["q.norm"], eps)
    k = norm(linear(x, w["k"]).view(T, g, d), w["k.norm"], eps)
    v = linear(x, w["v"]).view(T, g, dv)
    q = q * query_temperature(positions, m.get("q_temp"))[:, None, None]
    o = attend(q, k, v, m["scale"], visible(T), slopes=head_slopes(n))
    return linear(o.reshape(T, n * dv), w["o"])


# ---- gated linear attention --------------------------------------------------------------------------
def channel_decay(x, w, m):
    """[T, n, d]: sigmoid(a2 (a1 x) + b)^(1 / tau), one decay per head and key channel."""
    z = linear(linear(x, w["a1"]), w["a2"], w["a2.b"])
    return torch.sigmoid(z).pow(1.0 / float(m["tau"])).view(x.shape[0], m["heads"], m["dim"])


def linear_recurrence(q, k, v, decay, state=None):
    """Per head S <- diag(decay_t) S + k_t v_t^T, o_t = S^T q_t. q, k, decay [T, n, d], v [T, n, dv]; S [n, d, dv]
    starts at zero. Returns (o [T, n, dv], S)."""
    T, n, d = q.shape
    S = torch.zeros(n, d, v.shape[2], dtype=F64) if state is None else state.clone()
    out = torch.zeros(T, n, v.shape[2], dtype=F64)
    for t in range(T):
        S = decay[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("ndv,nd->nv", S, q[t])
    return out, S


def gated_linear_attention(x, w, m, eps):
    """The right side of the mixer 'parallel'."""
    T = x.shape[0]
    n, d, dv = m["heads"], m["dim"], m["vdim"]
    q = linear(x, w["q"]).view(T, n, d) * d ** -0.5
    k = linear(x, w["k"]).view(T, n, d)
    v = linear(x, w["v"]).view(T, n, dv)
    o, _ = linear_recurrence(q, k, v, channel_decay(x, w, m))
    o = norm(o, w["norm"], eps).reshape(T, n * dv) * silu(linear(x, w["g"]))
    return linear(o, w["o"])


def parallel_mixer(x, w, m, eps):
    return (m["left_scale"] * biased_attention(x, sub(w, "left."), m["left"], eps)
            + m["right_scale"] * gated_linear_attention(x, sub(w, "right."), m["right"], eps))


# ---- feed-forward -------------------------------------------------------------------------------------
def gated_ff(x, w):
    return linear(silu(linear(x, w["gate"])) * linear(x, w["up"]), w["down"])


def routed_experts(x, w, mlp):
    """Scores sigmoid(router x); a token's `top` best experts (the lower index on a tie) each run on score * x,
    and their results are added; the shared expert, where there is one, runs on x."""
    top = mlp["router"]["top"]
    scores = torch.sigmoid(linear(x, w["router"]))
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        order = sorted(range(scores.shape[1]), key=lambda e: (-float(scores[t, e]), e))[:top]
        for e in order:
            out[t] += gated_ff(scores[t, e] * x[t:t + 1], sub(w, f"e{e}."))[0]
    if mlp.get("shared"):
        out = out + gated_ff(x, sub(w, "shared."))
    return out


def feed_forward(x, w, mlp):
    return gated_ff(x, w) if mlp["kind"] == "dense" else routed_experts(x, w, mlp)


def sub(weights: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


# ---- the model ----------------------------------------------------------------------------------------
def forward(cfg: dict, weights: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the residual after every layer)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = len(tokens)
    eps = cfg["norm"]["eps"]
    positions = torch.arange(T)
    table = weights["embed"].to(F64)
    x = table[tokens] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    cached: dict[int, tuple] = {}
    seen = []
    for i, layer in enumerate(cfg["layers"]):
        m, mw = layer["mixer"], sub(weights, f"l{i}.mix.")
        if layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                cached[i] = keys_values(x, mw, m, eps, positions)
            y = window_attention(x, mw, m, eps, positions, kv=cached[i if src is None else src])
        elif layer["type"] == "parallel":
            y = parallel_mixer(x, mw, m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm(y, weights[f"l{i}.norm1"], eps)
        mlp = layer.get("mlp")
        if mlp:
            x = x + norm(feed_forward(x, sub(weights, f"l{i}.mlp."), mlp), weights[f"l{i}.norm2"], eps)
        seen.append(x.clone())
    logits = linear(norm(x, weights["final.norm"], eps), table) * float(cfg.get("logit_scale", 1.0))
    return (logits, torch.stack(seen)) if return_layers else logits
