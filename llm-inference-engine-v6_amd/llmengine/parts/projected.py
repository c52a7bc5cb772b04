"""Mixers of one shape: a single product of the layer's input with row-stacked matrices, a core
that turns the product's columns into activations, and a single output product. Several such
mixers that read the same input can then run side by side behind one input product and in front
of one output product (`ParallelMixer`).

A subclass names the matrices it stacks (`input_names`, each [rows, hidden]), the output matrix
(`output_name`, [hidden, out_width]), loads its small tensors in `load_core` and computes in
`core`. The stacked product's output is 32-bit; its columns are handed to the core as views.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import CacheSpec, Getter, LayerCache, Mixer, Placement
from .registry import register_part


def stack_rows(tensors: list[torch.Tensor], placement: Placement) -> tuple[torch.Tensor, int]:
    """The matrices one under the other on the device, rows padded with zeros to a multiple of 16 (so that
    the matrix kernels' blocked layout takes them). Returns (matrix, padded rows)."""
    dtype = placement.common_dtype(tensors)
    rows = sum(t.shape[0] for t in tensors)
    padded = (rows + 15) // 16 * 16
    fused = torch.zeros((padded, tensors[0].shape[1]), dtype=dtype, device=placement.device)
    at = 0
    for t in tensors:
        fused[at:at + t.shape[0]].copy_(t)
        at += t.shape[0]
    return placement.matrix(fused), padded


def stack_columns(tensors: list[torch.Tensor], placement: Placement) -> torch.Tensor:
    """Output matrices [hidden, k_i] side by side: one product over the concatenated activations adds
    what each would give."""
    dtype = placement.common_dtype(tensors)
    cols = sum(t.shape[1] for t in tensors)
    fused = torch.zeros((tensors[0].shape[0], cols), dtype=dtype, device=placement.device)
    at = 0
    for t in tensors:
        fused[:, at:at + t.shape[1]].copy_(t)
        at += t.shape[1]
    return placement.matrix(fused)


class ProjectedMixer(Mixer):
    graph_safe = True
    hidden_size: int
    out_width: int                      # columns of the core's result = inputs of the output matrix
    stacked_by_parent = False           # True: a parent stacks this mixer's matrices with others' and runs the products
    reads_foreign_cache = False         # True: the mixer keeps nothing itself and works on the cache another layer writes

    def input_names(self) -> list[tuple[str, int]]:
        """(local tensor name, rows) of the matrices that read the layer's input, in the order of the columns
        that `core` is given."""
        raise NotImplementedError

    def output_name(self) -> str:
        raise NotImplementedError

    @property
    def in_width(self) -> int:
        return sum(n for _, n in self.input_names())

    def load_core(self, get: Getter, placement: Placement) -> None:
        """The part's small tensors (everything but the stacked matrices)."""

    def core(self, p: torch.Tensor, step, cache: LayerCache | None, o: torch.Tensor, scale: float = 1.0) -> None:
        """p [T, in_width] 32-bit (a view with its own row stride) -> o [T, out_width] in the activation type
        (also a view), times `scale`."""
        raise NotImplementedError

    # ---- a mixer on its own ----
    def load_params(self, get: Getter, placement: Placement) -> None:
        if self.stacked_by_parent:          # (the parent has loaded the small tensors and stacked the matrices)
            return
        self.load_core(get, placement)
        self.w_in, self.in_padded = stack_rows([get(n) for n, _ in self.input_names()], placement)
        self.w_out = placement.place_matrix(get(self.output_name()))

    def forward(self, x, step, cache, out, accumulate, write_cache=True):
        if write_cache == self.reads_foreign_cache:
            raise NotImplementedError(f"{type(self).__name__} keeps a state of its own and cannot read another layer's"
                                      if not write_cache else f"{type(self).__name__} has nothing to write into a cache")
        T = x.shape[0]
        p = step.buffer("mixer.projected", (T, self.in_padded), torch.float32)
        ops.gemm(x, self.w_in, p, choices=step.choices)
        o = step.buffer("mixer.core_out", (T, self.out_width), step.act_dtype)
        self.core(p[:, :self.in_width], step, cache, o, 1.0)
        ops.gemm(o, self.w_out, out, accumulate, fixed_order=step.fixed_order, choices=step.choices)


class ParallelMixer(Mixer):
    """left_scale * left(x) + right_scale * right(x) for two projected mixers: one input product for both,
    their cores one after the other, one output product over both results side by side (each already
    times its scale)."""
    graph_safe = True

    def __init__(self, left: ProjectedMixer, right: ProjectedMixer, left_scale: float = 1.0, right_scale: float = 1.0,
                 names: tuple[str, str] = ("left", "right")):
        if left.hidden_size != right.hidden_size:
            raise ValueError("parallel mixers read the same input: their hidden sizes differ")
        self.sides = (left, right)
        self.scales = (float(left_scale), float(right_scale))
        self.side_names = tuple(names)
        self.hidden_size = left.hidden_size
        for side in self.sides:
            side.stacked_by_parent = True
        self._views: dict = {}

    def children(self):
        return dict(zip(self.side_names, self.sides))

    def refusals(self):
        return []

    def cache_spec(self) -> CacheSpec | None:
        paged, state, kind, window = {}, {}, "full", 0
        for name, side in zip(self.side_names, self.sides):
            spec = side.cache_spec()
            if spec is None:
                continue
            if spec.paged:
                if paged:
                    raise ValueError("parallel mixers: only one side may keep pages")
                kind, window = spec.kind, spec.window
            paged.update({f"{name}.{k}": v for k, v in spec.paged.items()})
            state.update({f"{name}.{k}": v for k, v in spec.state.items()})
        return CacheSpec(kind=kind, window=window, paged=paged, state=state) if (paged or state) else None

    def decode_round(self) -> int:
        return max(side.decode_round() for side in self.sides)

    def load_params(self, get: Getter, placement: Placement) -> None:
        ins, outs = [], []
        for name, side in zip(self.side_names, self.sides):
            side.load_core(lambda local, name=name: get(f"{name}.{local}"), placement)
            ins += [get(f"{name}.{n}") for n, _ in side.input_names()]
            outs.append(get(f"{name}.{side.output_name()}"))
        self.w_in, self.in_padded = stack_rows(ins, placement)
        self.w_out = stack_columns(outs, placement)

    def _side_cache(self, cache: LayerCache, name: str) -> LayerCache:
        key = (id(cache), name)
        view = self._views.get(key)
        if view is None or view[0] is not cache:
            pre = name + "."
            sub = LayerCache(paged={k[len(pre):]: t for k, t in cache.paged.items() if k.startswith(pre)},
                             state={k[len(pre):]: t for k, t in cache.state.items() if k.startswith(pre)},
                             page_size=cache.page_size, group=cache.group)
            if len(self._views) >= 64:
                self._views.clear()
            view = self._views[key] = (cache, sub)
        return view[1]

    def forward(self, x, step, cache, out, accumulate, write_cache=True):
        if not write_cache:
            raise NotImplementedError("parallel mixers keep states of their own and cannot read another layer's")
        T = x.shape[0]
        p = step.buffer("mixer.projected", (T, self.in_padded), torch.float32)
        ops.gemm(x, self.w_in, p, choices=step.choices)
        width = sum(side.out_width for side in self.sides)
        o = step.buffer("mixer.core_out", (T, width), step.act_dtype)
        col_in = col_out = 0
        for name, side, scale in zip(self.side_names, self.sides, self.scales):
            side.core(p[:, col_in:col_in + side.in_width], step, self._side_cache(cache, name),
                      o[:, col_out:col_out + side.out_width], scale)
            col_in += side.in_width
            col_out += side.out_width
        ops.gemm(o, self.w_out, out, accumulate, fixed_order=step.fixed_order, choices=step.choices)


register_part("mixer", "parallel", ParallelMixer)
