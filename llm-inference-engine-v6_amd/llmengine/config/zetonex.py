"""ZetonexConfig: the typed view of a Zetonex config.json.

The file names the vocabulary ("vocab"), the residual width ("width"), the norms' epsilon ("norm": {"eps"}), a
multiplier on the logits ("logit_scale"), optionally a stack of layers that runs several passes ("loop":
{"start", "stop", "times"}: layers start .. stop - 1 run `times` times in a row over the same weights) and a list
"layers", one entry per layer: "type" (which mixer), "mixer" (its sizes and constants) and "mlp" (the
feed-forward: "kind" "dense" with "ff", or "moe" with "router" {"experts", "top"} and "expert" {"ff", "limit"};
null for a layer without one). Nothing else is read. The design has no longest position and no end-of-sequence
token.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping

from .base import ConfigError, KeyReader

MIXER_TYPES = ("attention", "attention_2")
MLP_KINDS = ("dense", "moe")


@dataclass(frozen=True)
class ZetonexLayer:
    type: str
    mixer: Mapping[str, Any]            # the mixer's sizes and constants, checked, as plain values
    mlp: Mapping[str, Any] | None       # {"kind": "dense", "ff"} or {"kind": "moe", "experts", "top", "ff", "limit"}


def _rotation(m: KeyReader, dim: int) -> dict:
    rot = m.mapping("rot")
    if rot is None:
        return {"dims": 0, "base": 10000.0, "scaling": None}
    out = {"dims": rot.integer("dims", minimum=0), "base": rot.number("base"), "scaling": None}
    if out["dims"] % 2 or out["dims"] > dim:
        raise ConfigError(f"{rot.where}: dims={out['dims']} must be even and at most dim={dim}")
    if out["base"] <= 0:
        raise ConfigError(f"{rot.where}: base must be > 0")
    sc = rot.mapping("scaling")
    if sc is not None:
        out["scaling"] = {k: sc.number(k) for k in ("factor", "low", "high", "original")}
        if min(out["scaling"].values()) <= 0:
            raise ConfigError(f"{sc.where}: factor, low, high and original must be > 0")
    return out


def _mixer(r: KeyReader, kind: str) -> dict:
    m = r.mapping("mixer")
    if m is None:
        raise ConfigError(f"{r.where}: required key 'mixer' is missing")
    out = {"heads": m.integer("heads", minimum=1), "kv_heads": m.integer("kv_heads", minimum=1), "dim": m.integer("dim", minimum=1),
           "vdim": m.integer("vdim", minimum=1), "scale": m.number("scale"), "window": 0, "keep_first": 0}
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{m.where}: heads={out['heads']} is no multiple of kv_heads={out['kv_heads']}")
    out["rot"] = _rotation(m, out["dim"])
    mask = m.mapping("mask")
    if mask is not None:
        out["window"] = mask.integer("size", minimum=1)
        out["keep_first"] = mask.integer("keep_first", 0, minimum=0)
    if kind == "attention":
        if out["vdim"] != out["dim"]:
            raise ConfigError(f"{m.where}: the values of a mixer of type 'attention' are its keys: vdim={out['vdim']} must "
                              f"equal dim={out['dim']}")
    else:
        out["diff"] = m.number("diff")
        out["softcap"] = m.number("softcap", 0.0)
        if out["softcap"] < 0:
            raise ConfigError(f"{m.where}: softcap must be >= 0")
        if out["keep_first"]:
            raise ConfigError(f"{m.where}: a mixer of type 'attention_2' keeps no first tokens")
    return out


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
        out = {"kind": kind, "experts": router.integer("experts", minimum=1), "top": router.integer("top", minimum=1),
               "ff": expert.integer("ff", minimum=1), "limit": expert.number("limit")}
        if out["top"] > out["experts"]:
            raise ConfigError(f"{router.where}: top={out['top']} is more than experts={out['experts']}")
        if out["limit"] <= 0:
            raise ConfigError(f"{expert.where}: limit must be > 0")
        return out
    raise ConfigError(f"{mlp.where}: kind {kind!r} is none of {list(MLP_KINDS)}")


@dataclass(frozen=True)
class ZetonexConfig:
    architecture: str
    vocab_size: int
    width: int
    norm_eps: float
    logit_scale: float
    layers: tuple[ZetonexLayer, ...]
    loop: tuple[int, int, int] | None = None            # (start, stop, times)
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def max_pos(self) -> int:
        """Positions are not limited by the design (angles are computed from the position)."""
        return 1 << 30

    def layer_runs(self) -> list[tuple[int, int, bool]]:
        """(layer, pass, first of its pass) in the order the layers run: the layers in front of the loop once, the
        looped ones `times` times, then the rest."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, 0, False) for i in range(n)]
        start, stop, times = self.loop
        runs = [(i, 0, False) for i in range(start)]
        for p in range(times):
            runs += [(i, p, i == start) for i in range(start, stop)]
        return runs + [(i, 0, False) for i in range(stop, n)]

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], generation_cfg: Mapping[str, Any] | None = None,
                  architecture: str = "Zetonex") -> "ZetonexConfig":
        r = KeyReader(cfg)
        norm = r.mapping("norm")
        if norm is None:
            raise ConfigError("config.json: required key 'norm' is missing")
        raw = cfg.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: key 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw):
            lr = KeyReader(entry, f"config.json:layers[{i}]")
            kind = lr.string("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{lr.where}: mixer type {kind!r} is none of {list(MIXER_TYPES)}")
            layers.append(ZetonexLayer(kind, _mixer(lr, kind), _mlp(lr)))
        loop = None
        lp = r.mapping("loop")
        if lp is not None:
            loop = (lp.integer("start", minimum=0), lp.integer("stop", minimum=1), lp.integer("times", minimum=1))
            if not loop[0] < loop[1] <= len(layers):
                raise ConfigError(f"{lp.where}: start={loop[0]} and stop={loop[1]} must name a stretch of the {len(layers)} layers")
        return cls(architecture=architecture, vocab_size=r.integer("vocab", minimum=1), width=r.integer("width", minimum=1),
                   norm_eps=norm.number("eps"), logit_scale=r.number("logit_scale", 1.0), layers=tuple(layers), loop=loop)
