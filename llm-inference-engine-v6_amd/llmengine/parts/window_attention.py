"""Softmax attention over the paged cache with the variations that several designs put on it, each an argument:

* key and value sizes that differ (`dim`, `vdim`), grouped heads (query head h reads key/value head
  h // (heads // kv_heads));
* `values="keys"`: there is no value matrix; a value head is the key head as projected, before rotation;
* rotation of the first `rot_dims` entries of every query and key head, entry i with entry i + rot_dims / 2
  (`rot_pairs="halves"`) or entry 2 i with entry 2 i + 1 ("neighbours"), by position * f_i with
  f_i = rot_base^(-2 i / rot_dims), optionally stretched by wavelength band (`rot_scaling`: factor, low, high,
  original: waves shorter than original / high stay, waves longer than original / low slow down by the factor,
  between the two a linear blend in original / wavelength) or, with a factor alone, all slowed down by it;
* `qk_norm`: every query and key head is divided by its root mean square and multiplied by a weight over the
  head's entries ("q.norm", "k.norm", shared by all heads) before it is rotated;
* `softcap` > 0: score <- softcap * tanh(score / softcap);
* `window` > 0: a query at position p sees keys j with p - j < window, and with `keep_first` also the first
  keep_first tokens of the sequence, at their true positions;
* `gate`: the joined heads are multiplied element by element with sigmoid(Wg x) ("g") before the output matrix;
  `gate="heads"`: Wg has one row a head, and a head's whole result is multiplied by its one sigmoid;
* `sink`: a learned number per head ("sink") whose exponential joins the softmax's denominator: a key that is
  always visible, is not scaled and has no value;
* `q_temp=(coef, every)`: the queries of position p are multiplied by 1 + coef ln(floor((p + 1) / every) + 1);
* `distance_bias` = b > 0: the score of head h (from 0) loses 2^(-b (h + 1) / heads) for every token between query
  and key;
* `own_kv=False`: the layer has no key and value matrices (nor their norm): it reads the keys and values that
  another layer cached, with its own queries, window and everything else; `cache_window` is what the layer's own
  cache must keep where such readers look further back than the layer itself (0: everything);
* `maps=2` (differential attention): every head has two score maps with queries and keys of their own (rows of
  "q" and "k" head by head as [map 1, map 2]) over the same values; o = a_1 - lambda a_2 with
  lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, then o over its root mean square along the head's value
  entries, times (1 - diff).

Angles, norms, scores, weights and sums over keys are 32-bit; q and the cached k and v are kept in the activation
type. What is cached: k [kv_heads * maps, page, dim] after norm and rotation, v [kv_heads, vdim, page]. With a
window and nothing kept the cache gives pages back as the window passes; kept first tokens make it a full cache.
"""
from __future__ import annotations

import math

import torch

from .. import ops
from .base import PAGE, CacheSpec, Getter, ParamSpec, Placement
from .projected import ProjectedMixer
from .registry import register_part


def banded_frequencies(rot_dims: int, base: float, scaling: dict | None) -> torch.Tensor:
    """[rot_dims / 2] float64: base^(-2 i / rot_dims), stretched by wavelength band where `scaling` is given."""
    i = torch.arange(rot_dims // 2, dtype=torch.float64)
    freq = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / rot_dims)
    if scaling and "low" not in scaling:
        freq = freq / float(scaling["factor"])            # (every wave slowed down alike)
    elif scaling:
        factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        wave = 2.0 * math.pi / freq
        blend = (orig / wave - low) / (high - low) if high != low else torch.zeros_like(freq)
        mixed = (1.0 - blend) * freq / factor + blend * freq
        freq = torch.where(wave < orig / high, freq, torch.where(wave > orig / low, freq / factor, mixed))
    return freq


class WindowAttention(ProjectedMixer):
    def __init__(self, hidden_size: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, rot_dims: int = 0,
                 rot_base: float = 10000.0, rot_scaling: dict | None = None, window: int = 0, keep_first: int = 0,
                 softcap: float = 0.0, values: str = "projected", gate: bool | str = False, maps: int = 1, qk_norm: bool = False,
                 eps: float = 1e-6, diff: float = 0.0, rot_pairs: str = "halves", sink: bool = False,
                 q_temp: tuple[float, int] | None = None, distance_bias: float = 0.0, own_kv: bool = True,
                 cache_window: int | None = None):
        if heads % kv_heads:
            raise ValueError(f"{heads} query heads do not divide into {kv_heads} key/value heads")
        if rot_dims % 2 or not 0 <= rot_dims <= dim:
            raise ValueError(f"rot_dims {rot_dims} must be even and at most dim {dim}")
        if values not in ("projected", "keys"):
            raise ValueError(f"values {values!r} is neither 'projected' nor 'keys'")
        if values == "keys" and (vdim != dim or maps != 1):
            raise ValueError("values that are the keys need vdim == dim and one score map")
        if maps not in (1, 2):
            raise ValueError(f"maps={maps}: one score map a head, or two (differential attention)")
        if maps == 2 and gate:
            raise ValueError("the element-wise gate and two score maps do not go together")
        if window < 0 or keep_first < 0 or (keep_first and not window):
            raise ValueError("keep_first needs a window")
        if rot_pairs not in ("halves", "neighbours"):
            raise ValueError(f"rot_pairs {rot_pairs!r} is neither 'halves' nor 'neighbours'")
        if gate not in (False, True, "heads"):
            raise ValueError(f"gate {gate!r} is none of False, True (element by element) and 'heads'")
        if sink and maps != 1:
            raise ValueError("a sink goes with one score map a head")
        if not own_kv and values == "keys":
            raise ValueError("a layer that reads another's keys and values names no values of its own")
        if q_temp is not None and int(q_temp[1]) <= 0:
            raise ValueError("q_temp: the temperature steps every > 0 positions")
        if distance_bias < 0:
            raise ValueError("distance_bias must be >= 0")
        self.hidden_size = int(hidden_size)
        self.heads, self.kv_heads, self.dim, self.vdim = int(heads), int(kv_heads), int(dim), int(vdim)
        self.scale, self.softcap = float(scale), float(softcap)
        self.rot_dims, self.rot_base = int(rot_dims), float(rot_base)
        self.rot_scaling = dict(rot_scaling) if rot_scaling else None
        self.window, self.keep_first = int(window), int(keep_first)
        self.values, self.gate, self.maps, self.qk_norm = values, gate, int(maps), bool(qk_norm)
        self.rot_pairs, self.sink, self.own_kv = rot_pairs, bool(sink), bool(own_kv)
        self.q_temp = (float(q_temp[0]), int(q_temp[1])) if q_temp is not None else None
        self.distance_bias = float(distance_bias)
        self.reads_foreign_cache = not self.own_kv
        # what the cache keeps: the layer's own window unless told otherwise (0: everything)
        self.cache_window = self.window if cache_window is None else int(cache_window)
        self.sinks = self.slopes = None
        self.eps, self.diff = float(eps), float(diff)
        self.out_width = self.heads * self.vdim
        self.inv_freq: torch.Tensor | None = None
        self.wq = self.wk = None
        self.lam = 0.0

    # ---- tensors ----
    def input_names(self):
        n, g, M = self.heads, self.kv_heads, self.maps
        out = [("q", n * M * self.dim)]
        if self.own_kv:
            out.append(("k", g * M * self.dim))
            if self.values == "projected":
                out.append(("v", g * self.vdim))
        if self.gate:
            out.append(("g", n if self.gate == "heads" else n * self.vdim))
        return out

    def output_name(self):
        return "o"

    def param_specs(self):
        H = self.hidden_size
        out = {name: ParamSpec((rows, H)) for name, rows in self.input_names()}
        out["o"] = ParamSpec((H, self.out_width))
        if self.qk_norm:
            out["q.norm"] = ParamSpec((self.dim,), "norm")
            if self.own_kv:
                out["k.norm"] = ParamSpec((self.dim,), "norm")
        if self.sink:
            out["sink"] = ParamSpec((self.heads,))
        if self.maps == 2:
            out.update({k: ParamSpec((self.dim,)) for k in ("lq1", "lk1", "lq2", "lk2")})
        return out

    def refusals(self):
        if max(self.dim, self.vdim) > ops.window.WINDOW_ATTENTION_MAX_ENTRIES:
            return [f"dim={self.dim}, vdim={self.vdim}: the attention kernels hold heads of up to "
                    f"{ops.window.WINDOW_ATTENTION_MAX_ENTRIES} entries"]
        return []

    def cache_spec(self) -> CacheSpec | None:
        if not self.own_kv:
            return None
        slides = self.cache_window > 0 and self.keep_first == 0
        return CacheSpec(kind="window" if slides else "full", window=self.cache_window if slides else 0,
                         paged={"k": (self.kv_heads * self.maps, PAGE, self.dim), "v": (self.kv_heads, self.vdim, PAGE)})

    def load_core(self, get: Getter, placement: Placement) -> None:
        f32 = torch.float32
        if self.rot_dims:
            # frequencies in 64-bit, stored in 32-bit; the angle is the kernel's 32-bit product with the position
            self.inv_freq = placement.place(banded_frequencies(self.rot_dims, self.rot_base, self.rot_scaling).to(f32), f32)
        if self.qk_norm:
            self.wq = placement.place(get("q.norm"), f32)
            self.wk = placement.place(get("k.norm"), f32) if self.own_kv else None
        if self.sink:
            self.sinks = placement.place(get("sink"), f32)
        if self.distance_bias:
            h = torch.arange(1, self.heads + 1, dtype=torch.float64)
            self.slopes = placement.place(torch.pow(2.0, -self.distance_bias * h / self.heads).to(f32), f32)
        if self.maps == 2:
            l = {k: get(k).to(f32) for k in ("lq1", "lk1", "lq2", "lk2")}
            # one number for the layer, made once in 32-bit
            self.lam = float(torch.exp((l["lq1"] * l["lk1"]).sum()) - torch.exp((l["lq2"] * l["lk2"]).sum())
                             + torch.tensor(self.diff, dtype=f32))

    # ---- a step ----
    def core(self, p, step, cache, o, scale=1.0):
        T = p.shape[0]
        n, g, M, dim, vdim = self.heads, self.kv_heads, self.maps, self.dim, self.vdim
        nq = n * M
        own, projected = self.own_kv, self.values == "projected"
        k_col = nq * dim
        v_col = k_col + g * M * dim if own and projected else None
        g_col = nq * dim + ((g * M * dim + (g * vdim if projected else 0)) if own else 0)
        table = step.block_tables[cache.group]
        k_cache, v_cache = cache.paged["k"], cache.paged["v"]
        q = step.buffer("window_attention.q", (T, nq * dim), step.act_dtype)
        if own:
            ops.window.qk_prepare(p, step, table, q, k_cache, v_cache, nq, k_col, v_col, self.inv_freq, self.rot_dims,
                                  self.wq, self.wk, self.eps, self.rot_pairs, self.q_temp)
        else:
            ops.window.qk_prepare(p, step, None, q, None, None, nq, 0, None, self.inv_freq, self.rot_dims, self.wq, None,
                                  self.eps, self.rot_pairs, self.q_temp, dk=dim)
        # what is done with the runs' parts; where the keys are in one run the attention kernel may do it itself
        if M == 2:
            finish = dict(out=o, mode="difference", lam=self.lam, eps=self.eps, out_scale=(1.0 - self.diff) * scale)
        elif self.gate == "heads":
            finish = dict(out=o, mode="head_gate", gate=p[:, g_col:g_col + n], out_scale=scale, sinks=self.sinks)
        elif self.gate:
            finish = dict(out=o, mode="gate", gate=p[:, g_col:g_col + n * vdim], out_scale=scale, sinks=self.sinks)
        else:
            finish = dict(out=o, mode="plain", out_scale=scale, sinks=self.sinks)
        parts = ops.window.window_attention(q, k_cache, v_cache, step, table, nq, self.scale, self.softcap, self.window,
                                            self.keep_first, self.slopes, finish=finish)
        if parts != "finished":
            out = finish.pop("out")
            ops.window.window_attention_finish(parts[0], parts[1], out, n, **finish)


register_part("mixer", "window_attention", WindowAttention)
