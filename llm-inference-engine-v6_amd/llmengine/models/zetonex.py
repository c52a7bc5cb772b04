"""Zetonex as a list of layers and a schedule: layers whose mixer and feed-forward read one norm and add into the
stream together; two kinds of attention under sliding windows (one whose values are its keys, with kept first
tokens and an element-wise output gate; one with two score maps a head, normed queries and keys and capped scores);
a feed-forward that is dense with biases or a mixture of clamped experts chosen by a table over token ids; a stretch
of layers that may run several passes over the same weights, every pass with a cache of its own and an input map in
front of it; logits times a constant. Tensor names: "embed", "loop.in", "l<i>.norm1", "l<i>.mix.*", "l<i>.mlp.*",
"final.norm", "head".
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zetonex import ZetonexConfig, ZetonexLayer
from ..parts import make_part
from ..parts.reentry import PassInput
from .model import DecoderModel, LayerCall

_MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def zetonex_mixer(cfg: ZetonexConfig, layer: ZetonexLayer):
    m = layer.mixer
    common = dict(hidden_size=cfg.width, heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"], scale=m["scale"],
                  rot_dims=m["rot"]["dims"], rot_base=m["rot"]["base"], rot_scaling=m["rot"]["scaling"], window=m["window"],
                  keep_first=m["keep_first"], eps=cfg.norm_eps)
    if layer.type == "attention":
        return make_part("mixer", "window_attention", values="keys", gate=True, **common)
    return make_part("mixer", "window_attention", maps=2, qk_norm=True, softcap=m["softcap"], diff=m["diff"], **common)


def zetonex_feed_forward(cfg: ZetonexConfig, layer: ZetonexLayer):
    mlp = layer.mlp
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return make_part("feed_forward", "gated_mlp", hidden_size=cfg.width, intermediate_size=mlp["ff"], activation="silu",
                         names=_MLP_NAMES, bias=True)
    return make_part("feed_forward", "mixture_of_experts", hidden_size=cfg.width, intermediate_size=mlp["ff"],
                     experts=mlp["experts"], top=mlp["top"], activation="swish_clamped", limit=mlp["limit"], router="table",
                     vocab_size=cfg.vocab_size)


def build_zetonex(cfg: ZetonexConfig) -> DecoderModel:
    norm = lambda: make_part("norm", "rmsnorm_centered", size=cfg.width, eps=cfg.norm_eps, tensor="")
    layers = [make_part("block", "parallel", mixer=zetonex_mixer(cfg, layer), feed_forward=zetonex_feed_forward(cfg, layer),
                        mixer_norm=norm()) for layer in cfg.layers]
    # every run of a layer has a cache of its own: the first pass keeps the layer's number, later passes follow
    # behind the last layer's
    n = len(cfg.layers)
    span = (cfg.loop[1] - cfg.loop[0]) if cfg.loop else 0
    schedule = []
    for i, p, first in cfg.layer_runs():
        cache = i if p == 0 else n + (p - 1) * span + (i - cfg.loop[0])
        schedule.append(LayerCall(i, cache=cache, enter=first))
    embedding = make_part("embedding", "table", vocab_size=cfg.vocab_size, hidden_size=cfg.width, tensor="")
    head = make_part("head", "linear", vocab_size=cfg.vocab_size, hidden_size=cfg.width, tensor="", scale=cfg.logit_scale)
    return DecoderModel(cfg, embedding, layers, norm(), head, schedule=schedule,
                        pass_input=PassInput(cfg.width) if cfg.loop else None,
                        names={"embedding": "embed", "layers": "l{}", "final_norm": "final.norm", "head": "head",
                               "pass_input": "loop.in"})


register_architecture("Zetonex", ZetonexConfig.from_dict, build_zetonex)
