"""ZapolornConfig: the typed view of a Zapolorn config.json.

The file names the vocabulary ("vocab"), the residual width ("width"), a multiplier on the embedding ("embedding":
{"scale"}), the norms' epsilon ("norm": {"eps"}), a multiplier on the logits ("logit_scale") and a list "layers", one
entry per layer: "type" (which mixer), "mixer" (its sizes and constants) and "mlp" (the feed-forward: "kind" "dense"
with "ff", or "moe" with "router" {"experts", "top"}, "expert" {"ff"} and optionally "shared" {"ff"}; null for a
layer without one).

Mixer of type "attention": "heads", "kv_heads", "dim", "vdim", "scale", optionally "rot" {"base", "dims", "scaling"
{"factor"}}, "mask" {"size"} and "kv_from" (the layer whose keys and values this one reads). Mixer of type
"parallel": "left" {"heads", "kv_heads", "dim", "vdim", "scale", optionally "q_temp" {"coef", "every"}}, "right"
{"heads", "dim", "vdim", "tau"; "rank" only where random weights are made, a checkpoint's tensors give it},
"left_scale", "right_scale". Nothing else is read. The design has no longest position and no end-of-sequence token.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping

from .base import ConfigError, KeyReader

MIXER_TYPES = ("attention", "parallel")
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class ZapolornLayer:
    type: str
    mixer: Mapping[str, Any]            # the mixer's sizes and constants, checked, as plain values
    mlp: Mapping[str, Any] | None       # {"kind": "dense", "ff"} or {"kind": "moe", "experts", "top", "ff", "shared_ff"}


def _heads(m: KeyReader) -> dict:
    out = {"heads": m.integer("heads", minimum=1), "kv_heads": m.integer("kv_heads", minimum=1), "dim": m.integer("dim", minimum=1),
           "vdim": m.integer("vdim", minimum=1), "scale": m.number("scale")}
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{m.where}: heads={out['heads']} is no multiple of kv_heads={out['kv_heads']}")
    return out


def _attention(m: KeyReader) -> dict:
    out = _heads(m)
    out.update({"rot_dims": 0, "rot_base": 10000.0, "rot_factor": 1.0, "window": 0, "kv_from": None})
    rot = m.mapping("rot")
    if rot is not None:
        out["rot_dims"], out["rot_base"] = rot.integer("dims", minimum=0), rot.number("base")
        if out["rot_dims"] % 2 or out["rot_dims"] > out["dim"]:
            raise ConfigError(f"{rot.where}: dims={out['rot_dims']} must be even and at most dim={out['dim']}")
        if out["rot_base"] <= 0:
            raise ConfigError(f"{rot.where}: base must be > 0")
        sc = rot.mapping("scaling")
        if sc is not None:
            out["rot_factor"] = sc.number("factor")
            if out["rot_factor"] <= 0:
                raise ConfigError(f"{sc.where}: factor must be > 0")
    mask = m.mapping("mask")
    if mask is not None:
        out["window"] = mask.integer("size", minimum=1)
    if m.has("kv_from"):
        out["kv_from"] = m.integer("kv_from", minimum=0)
    return out


def _parallel(m: KeyReader) -> dict:
    left, right = m.mapping("left"), m.mapping("right")
    if left is None or right is None:
        raise ConfigError(f"{m.where}: a mixer of type 'parallel' needs 'left' and 'right'")
    lo = _heads(left)
    lo["q_temp"] = None
    qt = left.mapping("q_temp")
    if qt is not None:
        lo["q_temp"] = (qt.number("coef"), qt.integer("every", minimum=1))
    ro = {"heads": right.integer("heads", minimum=1), "dim": right.integer("dim", minimum=1),
          "vdim": right.integer("vdim", minimum=1), "tau": right.number("tau"),
          "rank": right.integer("rank", None, minimum=1) if right.has("rank") else None}
    if ro["tau"] <= 0:
        raise ConfigError(f"{right.where}: tau must be > 0")
    return {"left": lo, "right": ro, "left_scale": m.number("left_scale", 1.0), "right_scale": m.number("right_scale", 1.0)}


def _mlp(r: KeyReader) -> dict | None:
    mlp = r.mapping("mlp")
    if mlp is None:
        return None
    kind = mlp.string("kind")
    if kind == "dense":
        return {"kind": kind, "ff": mlp.integer("ff", minimum=1)}
    if kind == "moe":
        router, expert = mlp.mapping("router"), mlp.mapping("expert")
        if router is None or expert is None:
            raise ConfigError(f"{mlp.where}: a mixture of experts needs 'router' and 'expert'")
        shared = mlp.mapping("shared")
        out = {"kind": kind, "experts": router.integer("experts", minimum=1), "top": router.integer("top", minimum=1),
               "ff": expert.integer("ff", minimum=1), "shared_ff": shared.integer("ff", minimum=1) if shared is not None else None}
        if out["top"] > out["experts"]:
            raise ConfigError(f"{router.where}: top={out['top']} is more than experts={out['experts']}")
        return out
    raise ConfigError(f"{mlp.where}: kind {kind!r} is none of {list(MLP_KINDS)}")


@dataclass(frozen=True)
class ZapolornConfig:
    architecture: str
    vocab_size: int
    width: int
    embedding_scale: float
    norm_eps: float
    logit_scale: float
    layers: tuple[ZapolornLayer, ...]
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def max_pos(self) -> int:
        """Positions are not limited by the design (angles and biases are computed from the position)."""
        return 1 << 30

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], generation_cfg: Mapping[str, Any] | None = None,
                  architecture: str = "Zapolorn") -> "ZapolornConfig":
        r = KeyReader(cfg)
        norm = r.mapping("norm")
        if norm is None:
            raise ConfigError("config.json: required key 'norm' is missing")
        raw = cfg.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers: list[ZapolornLayer] = []
        for i, entry in enumerate(raw):
            lr = KeyReader(entry, f"config.json:layers[{i}]")
            kind = lr.string("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{lr.where}: mixer type {kind!r} is none of {list(MIXER_TYPES)}")
            m = lr.mapping("mixer")
            if m is None:
                raise ConfigError(f"{lr.where}: required key 'mixer' is missing")
            mixer = _attention(m) if kind == "attention" else _parallel(m)
            if kind == "attention" and mixer["kv_from"] is not None:
                j = mixer["kv_from"]
                if j >= i or layers[j].type != "attention" or layers[j].mixer["kv_from"] is not None:
                    raise ConfigError(f"{m.where}: kv_from={j} must name an earlier layer of type 'attention' with keys and "
                                      "values of its own")
                theirs = layers[j].mixer
                for key in ("kv_heads", "dim", "vdim", "rot_dims", "rot_base", "rot_factor"):
                    if theirs[key] != mixer[key]:
                        raise ConfigError(f"{m.where}: {key}={mixer[key]} differs from layer {j}'s {theirs[key]}, whose keys "
                                          "and values this layer reads")
            layers.append(ZapolornLayer(kind, mixer, _mlp(lr)))
        emb = r.mapping("embedding")
        return cls(architecture=architecture, vocab_size=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                   embedding_scale=emb.number("scale", 1.0) if emb is not None else 1.0, norm_eps=norm.number("eps"),
                   logit_scale=r.number("logit_scale", 1.0), layers=tuple(layers))
