"""Small Zetonex configurations for the tests, and weights for them that the tests draw themselves (matrices of
order one over the root of their inputs, norm weights around zero where the design stores them so, query and key
norm weights around one, biases of order a half, expert tables with distinct entries per row). `sharp` multiplies
an attention's scale so that its softmax stands on a few keys: a key that is lost, or one too many, then moves
the whole row."""
from __future__ import annotations

import json
import os

import torch


def gated(heads=4, kv_heads=2, dim=12, scale=0.3, base=50.0, dims=8, window=9, keep_first=3, mlp="dense", sharp=1.0):
    """The mixer whose values are its keys, with an element-wise output gate."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale * sharp}
    if dims:
        m["rot"] = {"base": base, "dims": dims}
    if window:
        m["mask"] = {"size": window}
        if keep_first:
            m["mask"]["keep_first"] = keep_first
    return {"type": "attention", "mixer": m, "mlp": feed_forward(mlp)}


def differential(heads=2, kv_heads=1, dim=10, vdim=14, scale=0.35, base=300.0, dims=6, scaling=True, window=7, softcap=30.0,
                 diff=0.2, mlp="moe", sharp=1.0):
    """The mixer with two score maps a head, normed queries and keys and capped scores."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale * sharp, "diff": diff}
    if softcap:
        m["softcap"] = softcap
    if dims:
        m["rot"] = {"base": base, "dims": dims}
        if scaling:
            m["rot"]["scaling"] = scaling if isinstance(scaling, dict) else {"factor": 3.0, "low": 1.0, "high": 5.0, "original": 40}
    if window:
        m["mask"] = {"size": window}
    return {"type": "attention_2", "mixer": m, "mlp": feed_forward(mlp)}


def feed_forward(kind, ff=24, experts=5, top=2, limit=1.25):
    if kind is None:
        return None
    if isinstance(kind, dict):
        return kind
    if kind == "dense":
        return {"kind": "dense", "ff": ff}
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}


def config(layers, width=28, vocab=61, eps=1e-5, logit_scale=1.5, loop=None):
    out = {"architecture": "Zetonex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
           "layers": list(layers)}
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


# both mixers, sizes that are no powers of two, a layer without feed-forward, a stretch of two layers in the middle
# that runs twice, layers in front of and behind it
MIXED = config([differential(window=11, mlp="dense"), gated(), differential(heads=3, kv_heads=3, dim=6, vdim=4, dims=4, scaling=None, mlp=None),
                gated(heads=3, kv_heads=1, dim=8, dims=8, window=13, keep_first=0, mlp=feed_forward("moe", experts=3, top=1)),
                differential(heads=1, dim=16, vdim=8, dims=0, window=20, softcap=0.0, mlp="dense")], loop=(1, 3, 2))
# sizes that the matrix kernels take (multiples of 16 and 32), as a model served in bfloat16 has them; the first
# two layers run three times
ALIGNED = config([gated(heads=4, kv_heads=2, dim=32, scale=0.15, base=10000.0, dims=16, window=40, keep_first=6,
                        mlp=feed_forward("moe", ff=64, experts=8, top=2)),
                  differential(heads=4, kv_heads=2, dim=32, vdim=48, scale=0.17, base=10000.0, dims=32,
                               scaling={"factor": 2.0, "low": 1.0, "high": 8.0, "original": 64}, window=24, softcap=20.0,
                               mlp={"kind": "dense", "ff": 128}),
                  gated(heads=8, kv_heads=1, dim=16, scale=0.25, dims=16, window=0, keep_first=0, mlp={"kind": "dense", "ff": 64})],
                 width=64, vocab=128, loop=(0, 2, 3))


def make_weights(cfg: dict, seed: int, dtype=torch.bfloat16) -> dict:
    """name -> tensor for every tensor of the configuration's model (names and shapes as the engine's model tree
    lists them; the values are the tests' own)."""
    from llmengine.config.registry import architecture_name, parse_config, resolve
    model = resolve(architecture_name(cfg)).build_model(parse_config(cfg))
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, spec in model.named_specs().items():
        shape = tuple(spec.shape)
        leaf = name.split(".")[-1]
        if leaf == "table":
            experts = int(spec.init.split(":")[1])
            out[name] = torch.stack([torch.randperm(experts, generator=g)[:shape[1]] for _ in range(shape[0])]).to(torch.int32)
            continue
        if name.endswith("q.norm") or name.endswith("k.norm"):
            t = torch.randn(shape, generator=g) * 0.2 + 1.0
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            t = torch.randn(shape, generator=g) * 0.3
        elif leaf == "b":
            t = torch.randn(shape, generator=g) * 0.5
        elif len(shape) == 1:
            t = torch.randn(shape, generator=g) * 0.25             # stored around zero
        elif name == "loop.in":
            # the stream passes and the embedding comes in again at a third
            w = shape[0]
            t = torch.cat([torch.eye(w), torch.eye(w) / 3.0], dim=1) + torch.randn(shape, generator=g) * 0.5 / w ** 0.5
        else:
            t = torch.randn(shape, generator=g) * 1.3 / shape[-1] ** 0.5
        out[name] = t.to(dtype)
    return out


def write_model(tmp_path, cfg: dict, seed: int, dtype=torch.bfloat16, weights: dict | None = None) -> tuple[str, dict]:
    from llmengine.weights import write_state_dict
    weights = weights if weights is not None else make_weights(cfg, seed, dtype)
    os.makedirs(str(tmp_path), exist_ok=True)
    with open(os.path.join(str(tmp_path), "config.json"), "w") as f:
        json.dump(cfg, f)
    write_state_dict(os.path.join(str(tmp_path), "model.safetensors"), weights)
    return str(tmp_path), weights
