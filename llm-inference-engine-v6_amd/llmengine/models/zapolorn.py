"""Zapolorn as a list of layers and a schedule: an embedding with a multiplier; layers whose sublayers read the stream
itself and are normed behind (x <- x + norm1(mixer(x)); x <- x + norm2(ff(x))); a windowed softmax attention with
normed and rotated queries and keys, a sink in the softmax and a sigmoid gate per head, which may read the keys and
values that an earlier layer cached; a pair of mixers side by side, a softmax attention over all earlier tokens whose
scores lose a slope per token of distance and whose queries grow with the position, and a gated linear attention
with a state per request; a feed-forward that is dense or a mixture of experts chosen by sigmoid scores that weigh
the experts' input, beside a shared expert; logits from the embedding table itself, times a constant. Tensor names:
"embed", "l<i>.norm1", "l<i>.mix.*", "l<i>.norm2", "l<i>.mlp.*", "final.norm".
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zapolorn import ZapolornConfig, ZapolornLayer
from ..parts import make_part
from .model import DecoderModel, LayerCall

_MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}
DISTANCE_BIAS = 8.0         # head h of n (from 0) loses 2^(-8 (h + 1) / n) per token of distance


def zapolorn_mixer(cfg: ZapolornConfig, layer: ZapolornLayer, keep: int):
    """keep: how many of the last tokens the layer's cache must hold (0: all), which is more than the layer's own
    window where a later layer reads the same keys through a wider one."""
    m = layer.mixer
    if layer.type == "attention":
        return make_part("mixer", "window_attention", hidden_size=cfg.width, heads=m["heads"], kv_heads=m["kv_heads"],
                         dim=m["dim"], vdim=m["vdim"], scale=m["scale"], rot_dims=m["rot_dims"], rot_base=m["rot_base"],
                         rot_scaling={"factor": m["rot_factor"]} if m["rot_factor"] != 1.0 else None, rot_pairs="neighbours",
                         window=m["window"], qk_norm=True, eps=cfg.norm_eps, sink=True, gate="heads",
                         own_kv=m["kv_from"] is None, cache_window=keep)
    lm, rm = m["left"], m["right"]
    left = make_part("mixer", "window_attention", hidden_size=cfg.width, heads=lm["heads"], kv_heads=lm["kv_heads"],
                     dim=lm["dim"], vdim=lm["vdim"], scale=lm["scale"], qk_norm=True, eps=cfg.norm_eps, q_temp=lm["q_temp"],
                     distance_bias=DISTANCE_BIAS)
    right = make_part("mixer", "gated_linear_attention", hidden_size=cfg.width, heads=rm["heads"], dim=rm["dim"],
                      vdim=rm["vdim"], tau=rm["tau"], eps=cfg.norm_eps, decay_rank=rm["rank"])
    return make_part("mixer", "parallel", left=left, right=right, left_scale=m["left_scale"], right_scale=m["right_scale"])


def zapolorn_feed_forward(cfg: ZapolornConfig, layer: ZapolornLayer):
    mlp = layer.mlp
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return make_part("feed_forward", "gated_mlp", hidden_size=cfg.width, intermediate_size=mlp["ff"], activation="silu",
                         names=_MLP_NAMES)
    shared = None
    if mlp["shared_ff"] is not None:
        shared = make_part("feed_forward", "gated_mlp", hidden_size=cfg.width, intermediate_size=mlp["shared_ff"],
                           activation="silu", names=_MLP_NAMES)
    return make_part("feed_forward", "mixture_of_experts", hidden_size=cfg.width, intermediate_size=mlp["ff"],
                     experts=mlp["experts"], top=mlp["top"], activation="silu", shared=shared, router="sigmoid",
                     weight_on="input")


def build_zapolorn(cfg: ZapolornConfig) -> DecoderModel:
    norm = lambda: make_part("norm", "rmsnorm", size=cfg.width, eps=cfg.norm_eps, tensor="")
    # what a layer's cache must keep: the widest window among the layers that read it (0, everything, wins)
    keep = {i: layer.mixer["window"] for i, layer in enumerate(cfg.layers)
            if layer.type == "attention" and layer.mixer["kv_from"] is None}
    for layer in cfg.layers:
        src = layer.mixer.get("kv_from") if layer.type == "attention" else None
        if src is not None:
            keep[src] = 0 if 0 in (keep[src], layer.mixer["window"]) else max(keep[src], layer.mixer["window"])
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        ff = zapolorn_feed_forward(cfg, layer)
        layers.append(make_part("block", "output_norm", mixer=zapolorn_mixer(cfg, layer, keep.get(i, 0)), feed_forward=ff,
                                mixer_norm=norm(), ffn_norm=norm() if ff is not None else None))
        src = layer.mixer.get("kv_from") if layer.type == "attention" else None
        schedule.append(LayerCall(i) if src is None else LayerCall(i, cache=src, write_cache=False))
    embedding = make_part("embedding", "table", vocab_size=cfg.vocab_size, hidden_size=cfg.width, tensor="",
                          scale=cfg.embedding_scale)
    head = make_part("head", "linear", vocab_size=cfg.vocab_size, hidden_size=cfg.width, tied_to=embedding, tensor="",
                     scale=cfg.logit_scale)
    return DecoderModel(cfg, embedding, layers, norm(), head, schedule=schedule,
                        names={"embedding": "embed", "layers": "l{}", "final_norm": "final.norm", "head": "head"})


register_architecture("Zapolorn", ZapolornConfig.from_dict, build_zapolorn)
