"""Gated feed-forward: down( act(gate(x)) * up(x) ); act is SiLU
(src/engine.cpp:213-217, src/kernels.cpp:26-31) unless the model names another. No biases unless `bias` is set:
then every product has one, stored as "<matrix name>.b".

Gate and up rows are stored interleaved in groups of 16 in one matrix, so that one
product yields both and a 16-column group of its output holds the gate and the up
value of the same 16 units next to each other.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import FeedForward, Getter, ParamSpec, Placement
from .registry import register_part


class GatedMLP(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu", names: dict | None = None,
                 bias: bool = False):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        if activation not in ops.GATE_ACTIVATIONS:
            raise ValueError(f"gated_mlp: activation {activation!r} is none of {sorted(ops.GATE_ACTIVATIONS)}")
        self.activation = activation
        self.bias = bool(bias)
        self.b_gate_up = self.b_down = None
        self.names = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
        if names:
            self.names.update(names)
        self.group = 16 if self.intermediate_size % 16 == 0 else self.intermediate_size
        self.w_gate_up: torch.Tensor | None = None
        self.w_down: torch.Tensor | None = None

    def param_specs(self):
        H, FF = self.hidden_size, self.intermediate_size
        n = self.names
        out = {n["gate"]: ParamSpec((FF, H)), n["up"]: ParamSpec((FF, H)), n["down"]: ParamSpec((H, FF))}
        if self.bias:
            out.update({n["gate"] + ".b": ParamSpec((FF,)), n["up"] + ".b": ParamSpec((FF,)), n["down"] + ".b": ParamSpec((H,))})
        return out

    def load_params(self, get: Getter, placement: Placement) -> None:
        H, FF, g = self.hidden_size, self.intermediate_size, self.group
        gate, up = get(self.names["gate"]), get(self.names["up"])
        dtype = placement.common_dtype([gate, up])
        fused = torch.empty((2 * FF, H), dtype=dtype, device=placement.device)
        view = fused.view(FF // g, 2, g, H)
        view[:, 0].copy_(gate.view(FF // g, g, H))
        view[:, 1].copy_(up.view(FF // g, g, H))
        self.w_gate_up = placement.matrix(fused)
        self.w_down = placement.place_matrix(get(self.names["down"]))
        if self.bias:
            # gate and up biases in the order of the fused matrix's rows
            bg, bu = get(self.names["gate"] + ".b"), get(self.names["up"] + ".b")
            both = torch.empty((FF // g, 2, g), dtype=placement.common_dtype([bg, bu]), device=placement.device)
            both[:, 0].copy_(bg.view(FF // g, g))
            both[:, 1].copy_(bu.view(FF // g, g))
            self.b_gate_up = both.view(2 * FF).contiguous()
            self.b_down = placement.place(get(self.names["down"] + ".b"))

    def fuses_norm(self, h, norm, step):
        # A few rows (decoding): one kernel applies the norm, both projections and the activation.
        rms = norm.fused_rms()
        return (rms is not None and not self.bias and self.group == 16 and self.activation == "silu" and step.act_dtype == torch.bfloat16
                and ops.gemv_norm_supported(h, rms[0], self.w_gate_up, h.shape[0], gated=True, choices=step.choices))

    def forward(self, x, step, out, accumulate, pre_norm=None):
        T = x.shape[0]
        FF = self.intermediate_size
        if pre_norm is not None:
            act = step.buffer("mlp.act", (T, FF), torch.bfloat16)
            weight, eps = pre_norm.fused_rms()
            ops.gemv_norm(x, weight, eps, self.w_gate_up, act, gated=True)
        elif self.bias:
            act = step.buffer("mlp.act", (T, FF), x.dtype)
            if self.activation != "silu" or not ops.gemm_gated_extra(x, self.w_gate_up, act, self.group, self.b_gate_up,
                                                                    choices=step.choices):
                # (few rows, or another type or activation) the product's 32-bit rows, then biases and activation in one pass
                gu = step.buffer("mlp.gate_up", (T, 2 * FF), torch.float32)
                ops.gemm(x, self.w_gate_up, gu, choices=step.choices)
                ops.window.gated_bias_act(gu, act, self.group, self.activation, self.b_gate_up)
        else:
            act = step.buffer("mlp.act", (T, FF), x.dtype)
            ops.gemm_gated(x, self.w_gate_up, act, self.group,
                           lambda shape, dtype: step.buffer("mlp.gate_up", shape, dtype), choices=step.choices,
                           activation=self.activation)
        ops.gemm(act, self.w_down, out, accumulate, fixed_order=step.fixed_order, choices=step.choices)
        if self.bias:
            ops.window.add_row_bias(out, self.b_down)


register_part("feed_forward", "gated_mlp", GatedMLP)
