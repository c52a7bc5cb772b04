"""Gated linear attention: a memory S [dim, vdim] per head that every token lets decay channel by channel,
writes its key and value into and then reads with its query:

    S <- diag(a_t) S + k_t v_t^T;    o_t = S^T q_t

q (times dim^-1/2), k (heads x dim) and v (heads x vdim) are projections of the input without biases. The decay is
one number per head and key channel, a = sigmoid(z)^(1 / tau) with z = Wa2 (Wa1 x) + b, a map through a small rank
that the checkpoint's tensors give ("a1" [rank, hidden], "a2" [heads * dim, rank], "a2.b"). Each head's o is divided
by its root mean square over vdim and multiplied by a weight of size vdim that the heads share ("norm"), the joined
heads by silu(Wg x); then the output matrix.

Kept per request: S, 32-bit, zero at admission. The decay (through its logarithm), the recurrence, the read-out norm
and the gate are 32-bit. The recurrence is the delta rule's kernel without the read before the write.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import CacheSpec, Getter, ParamSpec, Placement
from .projected import ProjectedMixer
from .registry import register_part


class GatedLinearAttention(ProjectedMixer):
    FUSED_DECAY_ROWS = 64           # steps of up to this many rows make the decay's logit inside the decay kernel

    def __init__(self, hidden_size: int, heads: int, dim: int, vdim: int, tau: float, eps: float, decay_rank: int | None = None):
        if not tau > 0:
            raise ValueError(f"gated linear attention: tau={tau} must be > 0")
        self.hidden_size = int(hidden_size)
        self.heads, self.dim, self.vdim = int(heads), int(dim), int(vdim)
        self.tau, self.eps = float(tau), float(eps)
        # the rank of the decay's two-stage map: named by the configuration, or read off the checkpoint's tensors
        self.decay_rank = int(decay_rank) if decay_rank is not None else None
        self.out_width = self.heads * self.vdim
        self.qkv_width = 2 * self.heads * self.dim + self.heads * self.vdim

    def input_names(self):
        qk, hv = self.heads * self.dim, self.heads * self.vdim
        return [("q", qk), ("k", qk), ("v", hv), ("g", hv), ("a1", self.decay_rank)]

    def output_name(self):
        return "o"

    def param_specs(self):
        H, qk, hv = self.hidden_size, self.heads * self.dim, self.heads * self.vdim
        return {"q": ParamSpec((qk, H)), "k": ParamSpec((qk, H)), "v": ParamSpec((hv, H)), "g": ParamSpec((hv, H)),
                "a1": ParamSpec((self.decay_rank, H)), "a2": ParamSpec((qk, self.decay_rank)), "a2.b": ParamSpec((qk,)),
                "norm": ParamSpec((self.vdim,), "norm"), "o": ParamSpec((H, hv))}

    def refusals(self):
        if self.dim > ops.recurrent.DELTA_MAX_DIM:
            return [f"dim={self.dim}: the recurrence kernel takes key sizes up to {ops.recurrent.DELTA_MAX_DIM}"]
        return []

    def cache_spec(self) -> CacheSpec:
        # (transposed: a column's key channels lie together, which is how the kernel's lanes hold them)
        return CacheSpec(state={"memory": ((self.heads, self.vdim, self.dim), torch.float32)})

    def load_core(self, get: Getter, placement: Placement) -> None:
        f32 = torch.float32
        a1, a2 = get("a1"), get("a2")
        if a1.shape[0] != a2.shape[1]:
            raise ValueError(f"gated linear attention: a1 {tuple(a1.shape)} and a2 {tuple(a2.shape)} disagree on the rank")
        self.decay_rank = int(a1.shape[0])
        self.a2 = placement.place(a2)
        self.a2_bias = placement.place(get("a2.b"), self.a2.dtype)
        self.norm_w = placement.place(get("norm"), f32)

    def core(self, p, step, cache, o, scale=1.0):
        T = p.shape[0]
        heads, dim, vdim = self.heads, self.dim, self.vdim
        C, hv = self.qkv_width, heads * vdim
        g_in = p[:, C:C + hv]
        decay = step.buffer("linear_attention.decay", (T, heads * dim), torch.float32)
        low_in = p[:, C + hv:C + hv + self.decay_rank]
        if T <= self.FUSED_DECAY_ROWS:
            # few rows: the second stage of the decay's map (a 32-bit sum over the rank), its bias and the decay in one kernel
            ops.sigmoid_decay(low_in, self.a2_bias, self.tau, decay, a2=self.a2)
        else:
            # many rows: the second stage as a product of its own, its 32-bit input made contiguous first
            low = step.buffer("linear_attention.decay_low", (T, self.decay_rank), torch.float32)
            ops.copy_cols(low_in, low)
            z = step.buffer("linear_attention.decay_in", (T, heads * dim), torch.float32)
            ops.gemm(low, self.a2, z, choices=step.choices)
            ops.sigmoid_decay(z, self.a2_bias, self.tau, decay)
        read = step.buffer("linear_attention.read", (T, hv), torch.float32)
        ops.delta_rule(p[:, :C], None, decay, cache.state["memory"], step, read, heads, heads, dim, vdim, per_channel=True,
                       q_scale=float(dim) ** -0.5)
        ops.gated_head_norm(read, self.norm_w, g_in, None, o, heads, vdim, self.eps, scale, activation="silu")


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
