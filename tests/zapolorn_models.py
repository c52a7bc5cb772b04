"""Small Zapolorn configurations for the tests, and weights for them that the tests draw themselves (matrices of
order one over the root of their inputs, norm weights around one, sinks and decay biases of order one, routers wide
enough that the experts' scores differ). `sharp` multiplies an attention's scale so that its softmax stands on a few
keys: a key that is lost, or one too many, then moves the whole row."""
from __future__ import annotations

import json
import os

import torch


def windowed(heads=6, kv_heads=2, dim=12, vdim=10, scale=0.3, base=50.0, dims=8, factor=2.0, window=9, kv_from=None, mlp="dense",
             sharp=1.0):
    """The mixer 'attention': a sliding window, a sink, a gate per head; `kv_from` names the layer whose keys it reads."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale * sharp}
    if dims:
        m["rot"] = {"base": base, "dims": dims}
        if factor:
            m["rot"]["scaling"] = {"factor": factor}
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": feed_forward(mlp)}


def parallel(heads=3, kv_heads=1, dim=10, vdim=6, scale=0.25, coef=0.4, every=5, r_heads=2, r_dim=6, r_vdim=9, tau=3.0, rank=4,
             left_scale=0.7, right_scale=1.3, mlp="moe", sharp=1.0):
    """The mixer 'parallel': attention over everything before with a bias by distance beside a gated linear attention."""
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale * sharp}
    if every:
        left["q_temp"] = {"coef": coef, "every": every}
    right = {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "tau": tau, "rank": rank}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": feed_forward(mlp)}


def feed_forward(kind, ff=24, experts=5, top=2, shared=14):
    if kind is None:
        return None
    if isinstance(kind, dict):
        return kind
    if kind == "dense":
        return {"kind": "dense", "ff": ff}
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def config(layers, width=28, vocab=61, eps=1e-5, logit_scale=0.6, embedding_scale=2.0):
    return {"architecture": "Zapolorn", "vocab": vocab, "width": width, "embedding": {"scale": embedding_scale},
            "norm": {"eps": eps}, "logit_scale": logit_scale, "layers": list(layers)}


# both mixers, sizes that are no powers of two, a layer without feed-forward, readers of another layer's keys with a
# wider and a narrower window than the writer's and not next to it, experts with and without a shared one
MIXED = config([windowed(window=11, mlp="dense"),
                parallel(),
                windowed(window=17, kv_from=0, mlp=None),
                windowed(heads=3, kv_heads=3, dim=8, vdim=14, dims=8, factor=0, window=13, mlp=feed_forward("moe", experts=3, top=1, shared=0)),
                windowed(window=5, kv_from=0, mlp=feed_forward("moe", ff=10, experts=4, top=3)),
                parallel(heads=2, kv_heads=2, dim=6, vdim=8, every=0, r_heads=3, r_dim=10, r_vdim=4, tau=1.0, rank=2, mlp="dense"),
                windowed(heads=3, kv_heads=3, dim=8, vdim=14, dims=8, factor=0, window=0, kv_from=3, mlp="dense")])
# sizes that the matrix kernels take (multiples of 16 and 32), as a model served in bfloat16 has them
ALIGNED = config([parallel(heads=4, kv_heads=2, dim=32, vdim=48, scale=0.1, coef=0.3, every=16, r_heads=4, r_dim=32, r_vdim=16, tau=8.0,
                           rank=8, mlp=feed_forward("moe", ff=64, experts=8, top=2, shared=32)),
                  windowed(heads=8, kv_heads=2, dim=32, vdim=16, scale=0.17, base=10000.0, dims=16, factor=4.0, window=40,
                           mlp={"kind": "dense", "ff": 128}),
                  windowed(heads=8, kv_heads=2, dim=32, vdim=16, scale=0.2, base=10000.0, dims=16, factor=4.0, window=24, kv_from=1,
                           mlp=feed_forward("moe", ff=32, experts=4, top=1, shared=0)),
                  parallel(heads=6, kv_heads=1, dim=64, vdim=32, scale=0.09, coef=0.6, every=64, r_heads=2, r_dim=40, r_vdim=24, tau=12.0,
                           rank=6, left_scale=1.2, right_scale=0.8, mlp={"kind": "dense", "ff": 64})],
                 width=64, vocab=128)


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
        if leaf == "sink":
            t = torch.randn(shape, generator=g) * 1.5
        elif name.endswith("a2.b"):
            t = torch.randn(shape, generator=g) + 1.5          # decays mostly near one, some that forget fast
        elif len(shape) == 1:
            t = torch.randn(shape, generator=g) * 0.2 + 1.0    # norm weights
        elif name == "embed":
            t = torch.randn(shape, generator=g) * 0.5
        elif leaf == "router":
            t = torch.randn(shape, generator=g) * 2.5 / shape[-1] ** 0.5
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
