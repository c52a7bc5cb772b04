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


def random_config(seed: int) -> dict:
    """A configuration drawn at random: two to six layers of both kinds in any order, head counts, sizes, windows and
    constants of many kinds (sizes the matrix kernels take and sizes they refuse), readers of earlier layers' keys,
    feed-forwards of every kind or none."""
    import random
    rng = random.Random(seed)

    def mlp():
        kind = rng.choice(["dense", "moe", "moe", None])
        if kind is None:
            return None
        if kind == "dense":
            return {"kind": "dense", "ff": rng.choice([40, 64, 100, 144])}
        experts = rng.choice([2, 3, 6, 10, 16])
        return feed_forward("moe", ff=rng.choice([16, 24, 48, 80]), experts=experts, top=rng.randint(1, min(experts, 4)),
                            shared=rng.choice([0, 32, 72]))

    layers, writers = [], []
    for i in range(rng.randint(2, 6)):
        if rng.random() < 0.6:
            if writers and rng.random() < 0.4:
                j = rng.choice(writers)
                m = dict(layers[j]["mixer"], kv_from=j, heads=layers[j]["mixer"]["kv_heads"] * rng.choice([1, 2, 3, 5]),
                         scale=rng.choice([0.1, 0.15, 0.22]))
                m.pop("mask", None)
                if rng.random() < 0.7:
                    m["mask"] = {"size": rng.randint(1, 180)}
            else:
                kv, dim = rng.choice([1, 2, 3, 4]), rng.choice([16, 24, 32, 40, 48, 64, 80, 96, 128])
                m = {"heads": kv * rng.choice([1, 2, 3, 4, 8]), "kv_heads": kv, "dim": dim, "vdim": rng.choice([16, 20, 32, 48, 64, 72, 96, 128]),
                     "scale": rng.choice([0.1, 0.15, 0.22, dim ** -0.5])}
                if rng.random() < 0.85:
                    m["rot"] = {"base": rng.choice([5000.0, 80000.0, 2e6]), "dims": rng.choice([dim, dim // 4 * 2, 8])}
                    if rng.random() < 0.7:
                        m["rot"]["scaling"] = {"factor": rng.choice([1.5, 4.0, 20.0])}
                if rng.random() < 0.85:
                    m["mask"] = {"size": rng.choice([1, 7, 16, 33, 64, 100, 129, 150, 240])}
                writers.append(i)
            layers.append({"type": "attention", "mixer": m, "mlp": mlp()})
        else:
            kv = rng.choice([1, 2, 4])
            layers.append(parallel(heads=kv * rng.choice([1, 2, 3, 4]), kv_heads=kv, dim=rng.choice([16, 32, 40, 64, 96, 128]),
                                   vdim=rng.choice([16, 24, 32, 64, 128]), scale=rng.choice([0.08, 0.11, 0.2]),
                                   coef=rng.choice([0.1, 0.3, 1.0]), every=rng.choice([0, 1, 16, 50, 100, 256]),
                                   r_heads=rng.choice([1, 2, 3, 5, 8]), r_dim=rng.choice([8, 16, 24, 40, 64, 100, 128]),
                                   r_vdim=rng.choice([8, 16, 32, 40, 64, 128]), tau=rng.choice([1.0, 4.0, 10.0, 50.0]),
                                   rank=rng.choice([3, 8, 16, 32]), left_scale=rng.choice([0.5, 0.9, 1.0]),
                                   right_scale=rng.choice([0.5, 1.0, 1.4]), mlp=mlp()))
    return config(layers, width=rng.choice([64, 96, 136, 160, 192, 320]), vocab=rng.choice([100, 257, 384]),
                  eps=rng.choice([1e-6, 1e-5]), logit_scale=rng.choice([0.3, 0.5, 1.0]), embedding_scale=rng.choice([1.0, 3.0, 8.0]))


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
            # (logits of order one whatever the embedding's multiplier: sigmoids that do not run into 0 or 1)
            t = torch.randn(shape, generator=g) * 2.5 / shape[-1] ** 0.5 / min(4.0, float(cfg.get("embedding", {}).get("scale", 1.0)))
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
