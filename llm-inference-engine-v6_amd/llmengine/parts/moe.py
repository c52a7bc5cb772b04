"""Mixture of experts: a router scores E small gated feed-forward layers for every token, the token runs
the `top` best of them, and their results are added with the router's weights; a shared expert of the same
form may run for every token beside them.

Router: z = Wr x in 32-bit (the matrix is kept in 32-bit), s = softmax(z) over all experts, the `top`
largest s are chosen (the lower index wins a tie), weight = s * scale, divided by the chosen scores' sum
first where `renormalize` is set. Expert e: down_e(act(gate_e x) * up_e x), no biases. Tensors: "router",
"e<i>.gate", "e<i>.up", "e<i>.down"; the shared expert is a child part under "shared".

`router="sigmoid"`: the scores are sigmoid(z), each expert's on its own, and the largest are chosen.
`weight_on="input"`: a chosen expert runs on weight * x and its result is added as it is (the weight is taken out of
the expert's two input products: their 32-bit sums are multiplied by it in front of the activation).

`router="table"`: there is no router matrix; a table [vocab, top] of integers ("table"; the entries of a row differ)
names the experts of every token id, each weighing 1 / top. `activation="swish_clamped"` with `limit`:
g = min(gate, limit), u = clamp(up, -limit, limit), the expert's inner value is g sigmoid(1.702 g) (u + 1).

On the device the (token, expert) pairs are grouped by expert into tiles of rows, and two grouped products
(gate/up with the activation, then down) run over the tiles; nothing of the routing comes to the host, so
a step's launches do not depend on what the tokens choose.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import FeedForward, Getter, ParamSpec, Placement
from .registry import register_part


class MixtureOfExperts(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, experts: int, top: int, scale: float = 1.0,
                 renormalize: bool = False, activation: str = "silu", shared: FeedForward | None = None,
                 expert_name: str = "e{}", router: str = "softmax", vocab_size: int = 0, limit: float = 0.0,
                 weight_on: str = "output"):
        if router not in ("softmax", "sigmoid", "table"):
            raise ValueError(f"mixture_of_experts: router {router!r} is none of 'softmax', 'sigmoid' and 'table'")
        if weight_on not in ("output", "input"):
            raise ValueError(f"mixture_of_experts: weight_on {weight_on!r} is neither 'output' nor 'input'")
        if weight_on == "input" and activation == "swish_clamped":
            raise ValueError("mixture_of_experts: weights on the experts' input do not go with the clamped activation")
        if router == "table" and vocab_size <= 0:
            raise ValueError("mixture_of_experts: a table of experts by token id needs vocab_size")
        if not 1 <= top <= experts:
            raise ValueError(f"top={top} must be between 1 and experts={experts}")
        if activation not in ops.GATE_ACTIVATIONS and activation != "swish_clamped":
            raise ValueError(f"mixture_of_experts: activation {activation!r} is none of "
                             f"{sorted(ops.GATE_ACTIVATIONS) + ['swish_clamped']}")
        if activation == "swish_clamped" and not limit > 0:
            raise ValueError("mixture_of_experts: the clamped activation needs limit > 0")
        self.router, self.vocab_size, self.limit = router, int(vocab_size), float(limit)
        self.weight_on = weight_on
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.experts, self.top, self.scale = int(experts), int(top), float(scale)
        self.renormalize, self.activation = bool(renormalize), activation
        self.shared, self.expert_name = shared, expert_name

    def children(self):
        return {"shared": self.shared} if self.shared is not None else {}

    def refusals(self):
        if self.experts > ops.latent.MOE_MAX_EXPERTS:
            return [f"experts={self.experts}: the routing kernels take up to {ops.latent.MOE_MAX_EXPERTS}"]
        return []

    def param_specs(self):
        H, FF = self.hidden_size, self.intermediate_size
        out = ({"router": ParamSpec((self.experts, H))} if self.router != "table"
               else {"table": ParamSpec((self.vocab_size, self.top), f"table:{self.experts}")})
        for e in range(self.experts):
            name = self.expert_name.format(e)
            out.update({f"{name}.gate": ParamSpec((FF, H)), f"{name}.up": ParamSpec((FF, H)), f"{name}.down": ParamSpec((H, FF))})
        return out

    def load_params(self, get: Getter, placement: Placement) -> None:
        # The router's matrix as the file has it: bfloat16 entries times the bfloat16 input are exact in 32-bit, so the
        # matrix-core product with its 32-bit sums is the 32-bit product; the 32-bit model widens it like everything else.
        if self.router != "table":
            self.w_router = placement.place(get("router"))
        else:
            self.table = placement.place(get("table"))
            if int(self.table.min()) < 0 or int(self.table.max()) >= self.experts:
                raise ValueError(f"mixture_of_experts: the table names experts outside 0..{self.experts - 1}")
        E, FF, H = self.experts, self.intermediate_size, self.hidden_size
        names = [self.expert_name.format(e) for e in range(E)]
        dtype = placement.common_dtype([get(f"{names[0]}.{k}") for k in ("gate", "up", "down")])
        # gate and up rows of an expert in alternating groups of 16 in one matrix, as the dense feed-forward keeps them
        g = self.group = 16 if FF % 16 == 0 else FF
        self.w_gate_up = torch.empty((E, 2 * FF, H), dtype=dtype, device=placement.device)
        view = self.w_gate_up.view(E, FF // g, 2, g, H)
        for e, name in enumerate(names):
            view[e, :, 0].copy_(get(f"{name}.gate").view(FF // g, g, H))
            view[e, :, 1].copy_(get(f"{name}.up").view(FF // g, g, H))
        self.w_down = torch.stack([placement.place(get(f"{n}.down"), dtype) for n in names]).contiguous()

    def forward(self, x, step, out, accumulate):
        T, H = x.shape
        E, top, FF = self.experts, self.top, self.intermediate_size
        i32, f32 = torch.int32, torch.float32
        ids, wts = step.buffer("moe.ids", (T, top), i32), step.buffer("moe.weights", (T, top), f32)
        if self.router == "table":
            ops.window.table_route(self.table, step.tokens, ids, wts)
        else:
            logits = step.buffer("moe.logits", (T, E), f32)
            ops.gemm(x, self.w_router, logits, choices=step.choices)
            ops.moe_route(logits, top, self.scale, self.renormalize, ids, wts, scoring=self.router)
        tile = ops.latent.moe_tile(x, self.w_gate_up, T * top, E, self.group, step.choices)
        cap = ops.moe_capacity(T * top, E, tile)
        place_pair, pair_place = step.buffer("moe.place_pair", (cap,), i32), step.buffer("moe.pair_place", (T * top,), i32)
        tile_expert, n_tiles = step.buffer("moe.tile_expert", (cap // tile,), i32), step.buffer("moe.tiles", (1,), i32)
        ops.moe_plan(ids, E, tile, place_pair, pair_place, tile_expert, n_tiles)
        act = step.buffer("moe.act", (cap, FF), step.act_dtype)
        if self.activation == "swish_clamped" and ops.latent.moe_gemm_clamped(x, self.w_gate_up, self.group, act, place_pair,
                                                                             tile_expert, n_tiles, tile, top, self.limit, 1.702,
                                                                             step.choices):
            pass                            # (clamps and activation in the product's epilogue)
        elif self.weight_on == "input" and self.activation == "silu" and ops.latent.moe_gemm_clamped(
                x, self.w_gate_up, self.group, act, place_pair, tile_expert, n_tiles, tile, top, 0.0, 1.0, step.choices,
                pair_scale=wts.view(-1)):
            pass                            # (a place's sums times its pair's weight, then the activation, in the product's epilogue)
        elif self.weight_on == "input":
            # the gate and up sums as 32-bit rows, each row times its pair's weight, then the activation, in one pass
            gu = step.buffer("moe.gate_up", (cap, 2 * FF), f32)
            ops.moe_gemm(x, self.w_gate_up, False, 0, gu, place_pair, tile_expert, n_tiles, tile, top, "silu", step.choices)
            ops.window.gated_bias_act(gu, act, self.group, self.activation, row_pair=place_pair, pair_scale=wts.view(-1))
        elif self.activation == "swish_clamped":
            # the gate and up columns as 32-bit rows, then clamps and activation in one pass
            gu = step.buffer("moe.gate_up", (cap, 2 * FF), f32)
            ops.moe_gemm(x, self.w_gate_up, False, 0, gu, place_pair, tile_expert, n_tiles, tile, top, "silu", step.choices)
            ops.window.gated_bias_act(gu, act, self.group, "swish_clamped", None, self.limit, 1.702)
        else:
            ops.moe_gemm(x, self.w_gate_up, True, self.group, act, place_pair, tile_expert, n_tiles, tile, top, self.activation,
                         step.choices)
        y = step.buffer("moe.y", (cap, H), f32)
        ops.moe_gemm(act, self.w_down, False, 0, y, place_pair, tile_expert, n_tiles, tile, 0, "silu", step.choices)
        if self.shared is not None:
            self.shared.forward(x, step, out, accumulate)
            accumulate = True
        ops.moe_combine(y, pair_place, wts if self.weight_on == "output" else None, out, accumulate, top=top)


register_part("feed_forward", "mixture_of_experts", MixtureOfExperts)
