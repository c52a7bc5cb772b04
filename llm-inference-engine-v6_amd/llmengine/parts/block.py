"""Arrangement of a layer's parts around the residual stream.

Pre-norm (src/engine.cpp:137-239): h += mixer(norm1(h)); h += ffn(norm2(h)). The
residual stream h is 32-bit; mixer and feed-forward add their result into it
(their last product accumulates into h), so the sum is made in 32-bit.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Block, FeedForward, Mixer, Norm
from .registry import register_part


class PreNormBlock(Block):
    graph_safe = True

    def __init__(self, mixer: Mixer, feed_forward: FeedForward | None, mixer_norm: Norm, ffn_norm: Norm | None,
                 names: dict | None = None):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.ffn_norm = mixer_norm, ffn_norm
        # Names under which a checkpoint stores this layer's parts.
        self.names = {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                      "ffn_norm": "post_attention_layernorm", "feed_forward": "mlp"}
        if names:
            self.names.update(names)

    def children(self):
        n = self.names
        out = {n["mixer_norm"]: self.mixer_norm, n["mixer"]: self.mixer}
        if self.feed_forward is not None:
            out.update({n["ffn_norm"]: self.ffn_norm, n["feed_forward"]: self.feed_forward})
        return out

    def forward(self, h, step, cache, write_cache=True):
        T, H = h.shape
        x = step.buffer("block.normed", (T, H), step.act_dtype)
        if self.mixer.fuses_norm(h, self.mixer_norm, step):
            self.mixer.forward(h, step, cache, h, True, write_cache, pre_norm=self.mixer_norm)
        else:
            self.mixer_norm.forward(h, x)
            self.mixer.forward(x, step, cache, h, True, write_cache)
        if self.feed_forward is None:
            return
        if self.feed_forward.fuses_norm(h, self.ffn_norm, step):
            self.feed_forward.forward(h, step, h, True, pre_norm=self.ffn_norm)
        else:
            self.ffn_norm.forward(h, x)
            self.feed_forward.forward(x, step, h, True)


class SandwichBlock(Block):
    """A norm in front of and behind every sublayer: h += post1(mixer(pre1(h))); h += post2(ffn(pre2(h))).
    A sublayer's result is a 32-bit buffer of its own; the norm behind it, the sum into the stream and the
    norm in front of whatever reads the stream next (this block's feed-forward, or the first sublayer of
    the block behind) are one kernel where all three norms are the plain RMS formula."""
    graph_safe = True

    def __init__(self, mixer: Mixer, feed_forward: FeedForward | None, mixer_norm: Norm, ffn_norm: Norm | None,
                 mixer_post_norm: Norm, ffn_post_norm: Norm | None, names: dict | None = None):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.ffn_norm = mixer_norm, ffn_norm
        self.mixer_post_norm, self.ffn_post_norm = mixer_post_norm, ffn_post_norm
        self.names = {"mixer_norm": "norm1", "mixer": "mix", "mixer_post_norm": "norm1b",
                      "ffn_norm": "norm2", "feed_forward": "mlp", "ffn_post_norm": "norm2b"}
        if names:
            self.names.update(names)
        # the block that runs behind this one (told by the model as it runs its schedule; None: unknown)
        self.next_block = None

    def children(self):
        n = self.names
        out = {n["mixer_norm"]: self.mixer_norm, n["mixer_post_norm"]: self.mixer_post_norm, n["mixer"]: self.mixer}
        if self.feed_forward is not None:
            out.update({n["ffn_norm"]: self.ffn_norm, n["ffn_post_norm"]: self.ffn_post_norm,
                        n["feed_forward"]: self.feed_forward})
        return out

    def _join(self, y, post: Norm, h, nxt: Norm | None, x, step) -> bool:
        """h += post(y); True if x was also made = nxt(h)."""
        rms = post.fused_rms()
        nxt_rms = nxt.fused_rms() if nxt is not None else None
        if rms is not None and nxt_rms is not None and nxt_rms[0].dtype == rms[0].dtype and nxt_rms[1] == rms[1]:
            ops.norm_add(y, rms[0], h, rms[1], nxt_rms[0], x)
            return True
        if rms is not None:
            ops.norm_add(y, rms[0], h, rms[1])
        else:
            raise NotImplementedError("sandwich blocks take norms of the plain RMS formula behind their sublayers")
        return False

    def forward(self, h, step, cache, write_cache=True):
        T, H = h.shape
        x = step.buffer("block.normed", (T, H), step.act_dtype)
        y = step.buffer("block.sublayer", (T, H), torch.float32)
        if step.extra.pop("block.normed is for", None) != id(self):
            self.mixer_norm.forward(h, x)
        self.mixer.forward(x, step, cache, y, False, write_cache)
        behind = self.next_block.mixer_norm if isinstance(self.next_block, SandwichBlock) else None
        if self.feed_forward is None:
            if self._join(y, self.mixer_post_norm, h, behind, x, step):
                step.extra["block.normed is for"] = id(self.next_block)
            return
        if not self._join(y, self.mixer_post_norm, h, self.ffn_norm, x, step):
            self.ffn_norm.forward(h, x)
        self.feed_forward.forward(x, step, y, False)
        if self._join(y, self.ffn_post_norm, h, behind, x, step):
            step.extra["block.normed is for"] = id(self.next_block)


class ParallelBlock(Block):
    """One norm whose output both sublayers read: h += mixer(norm(h)) + ffn(norm(h)). Both sublayers add into the
    32-bit stream (their last products accumulate), the mixer first."""
    graph_safe = True

    def __init__(self, mixer: Mixer, feed_forward: FeedForward | None, mixer_norm: Norm, ffn_norm: Norm | None = None,
                 names: dict | None = None):
        if ffn_norm is not None:
            raise ValueError("a parallel block has one norm: its feed-forward reads the mixer's")
        self.mixer, self.feed_forward, self.mixer_norm = mixer, feed_forward, mixer_norm
        self.names = {"mixer_norm": "norm1", "mixer": "mix", "feed_forward": "mlp"}
        if names:
            self.names.update(names)

    def children(self):
        n = self.names
        out = {n["mixer_norm"]: self.mixer_norm, n["mixer"]: self.mixer}
        if self.feed_forward is not None:
            out[n["feed_forward"]] = self.feed_forward
        return out

    def forward(self, h, step, cache, write_cache=True):
        T, H = h.shape
        x = step.buffer("block.normed", (T, H), step.act_dtype)
        self.mixer_norm.forward(h, x)
        self.mixer.forward(x, step, cache, h, True, write_cache)
        if self.feed_forward is not None:
            self.feed_forward.forward(x, step, h, True)


class OutputNormBlock(Block):
    """Norms behind the sublayers only: h += norm1(mixer(h)); h += norm2(ffn(h)). The sublayers read the stream itself
    (rounded to the activation type where that is not 32-bit); a sublayer's result is a 32-bit buffer of its own, and
    the norm behind it, the sum into the stream and the copy of the updated rows that the next sublayer reads (this
    block's feed-forward, or the mixer of the block behind) are one kernel."""
    graph_safe = True

    def __init__(self, mixer: Mixer, feed_forward: FeedForward | None, mixer_norm: Norm, ffn_norm: Norm | None,
                 names: dict | None = None):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.ffn_norm = mixer_norm, ffn_norm
        self.names = {"mixer_norm": "norm1", "mixer": "mix", "ffn_norm": "norm2", "feed_forward": "mlp"}
        if names:
            self.names.update(names)
        # the block that runs behind this one (told by the model as it runs its schedule; None: unknown)
        self.next_block = None

    def children(self):
        n = self.names
        out = {n["mixer_norm"]: self.mixer_norm, n["mixer"]: self.mixer}
        if self.feed_forward is not None:
            out.update({n["ffn_norm"]: self.ffn_norm, n["feed_forward"]: self.feed_forward})
        return out

    @staticmethod
    def _join(y, post: Norm, h, x) -> None:
        """h += post(y), and x = the updated rows where x is another buffer than the stream."""
        rms = post.fused_rms()
        if rms is None:
            raise NotImplementedError("output-norm blocks take norms of the plain RMS formula behind their sublayers")
        ops.norm_add(y, rms[0], h, rms[1], None, x if x is not h else None)

    def forward(self, h, step, cache, write_cache=True):
        T, H = h.shape
        y = step.buffer("block.sublayer", (T, H), torch.float32)
        if step.act_dtype == torch.float32:
            x = h                           # (the sublayers read the 32-bit stream as it lies)
        else:
            x = step.buffer("block.stream_copy", (T, H), step.act_dtype)
            if step.extra.pop("block.stream_copy is for", None) != id(self):
                ops.copy_cols(h, x)
        self.mixer.forward(x, step, cache, y, False, write_cache)
        hand_on = isinstance(self.next_block, OutputNormBlock) and x is not h
        if self.feed_forward is None:
            self._join(y, self.mixer_norm, h, x if hand_on else h)
        else:
            self._join(y, self.mixer_norm, h, x)
            self.feed_forward.forward(x, step, y, False)
            self._join(y, self.ffn_norm, h, x if hand_on else h)
        if hand_on:
            step.extra["block.stream_copy is for"] = id(self.next_block)


register_part("block", "prenorm", PreNormBlock)
register_part("block", "output_norm", OutputNormBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "sandwich", SandwichBlock)
