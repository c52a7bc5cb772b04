"""The map that a stack of layers run several times in a row puts in front of every pass: the stream so far and the
embedding's output side by side, through one matrix [width, 2 width] (the stream's columns first), become the
pass's input, x <- W [x; x0]. The two rows are joined in the activation type and multiplied as one product with a
32-bit result."""
from __future__ import annotations

import torch

from .. import ops
from .base import Getter, ParamSpec, Part, Placement


class PassInput(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, tensor: str = ""):
        self.hidden_size = int(hidden_size)
        self.tensor = tensor
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        return {self.tensor: ParamSpec((self.hidden_size, 2 * self.hidden_size))}

    def load_params(self, get: Getter, placement: Placement) -> None:
        self.weight = placement.place_matrix(get(self.tensor))

    def forward(self, h: torch.Tensor, h0: torch.Tensor, step) -> None:
        """h [T, H] (32-bit, replaced) from h and the embedding's output h0."""
        T, H = h.shape
        both = step.buffer("pass_input.both", (T, 2 * H), step.act_dtype)
        ops.window.concat_rows(h, h0, both)
        ops.gemm(both, self.weight, h, choices=step.choices)
