"""Arrangement of a layer's parts around the residual stream.

Pre-norm (src/engine.cpp:137-239): h += mixer(norm1(h)); h += ffn(norm2(h)). The
residual stream h is 32-bit; mixer and feed-forward add their result into it
(their last product accumulates into h), so the sum is made in 32-bit.
"""
from __future__ import annotations

from .base import Block, FeedForward, Mixer, Norm
from .registry import register_part


class PreNormBlock(Block):
    graph_safe = True

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, ffn_norm: Norm,
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
        return {n["mixer_norm"]: self.mixer_norm, n["mixer"]: self.mixer,
                n["ffn_norm"]: self.ffn_norm, n["feed_forward"]: self.feed_forward}

    def forward(self, h, step, cache, write_cache=True):
        T, H = h.shape
        x = step.buffer("block.normed", (T, H), step.act_dtype)
        if self.mixer.fuses_norm(h, self.mixer_norm, step):
            self.mixer.forward(h, step, cache, h, True, write_cache, pre_norm=self.mixer_norm)
        else:
            self.mixer_norm.forward(h, x)
            self.mixer.forward(x, step, cache, h, True, write_cache)
        if self.feed_forward.fuses_norm(h, self.ffn_norm, step):
            self.feed_forward.forward(h, step, h, True, pre_norm=self.ffn_norm)
        else:
            self.ffn_norm.forward(h, x)
            self.feed_forward.forward(x, step, h, True)


register_part("block", "prenorm", PreNormBlock)
