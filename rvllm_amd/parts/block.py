"""Arrangements of norm, mixer, feed-forward and residual sum in a layer.

``sandwich``: a norm before and after each branch; the normed branch output
is added to the residual stream
(v3/crates/rvllm-loader/src/metal_host.rs:501,606-628; the order of launches:
v3/crates/rvllm-runtime/src/gemma4_layer_exec.rs:1-28):

    x = x + post_attention_layernorm(mixer(input_layernorm(x)))
    x = x + post_feedforward_layernorm(ff(pre_feedforward_layernorm(x)))

A block may hand the next block its entry norm already applied (``then``),
which lets the kernel that adds the feed-forward branch also write the next
layer's normed input.
"""

from __future__ import annotations

from typing import Optional

import torch

from .base import Block, Norm, ParamSpec
from .registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS
from .spec import LayerSpec, PartSpec


class SandwichBlock(Block):
    NORM_NAMES = ("input_layernorm", "post_attention_layernorm", "pre_feedforward_layernorm",
                  "post_feedforward_layernorm")

    def __init__(self, spec: PartSpec, *, layer: LayerSpec, hidden_size: int):
        self.hidden_size = hidden_size
        self.mixer = MIXERS.build(layer.mixer, hidden_size=hidden_size)
        self.feed_forward = FEED_FORWARDS.build(layer.feed_forward, hidden_size=hidden_size)
        self.norm_in, self.norm_post_mixer, self.norm_pre_ff, self.norm_post_ff = (
            NORMS.build(layer.norm, width=hidden_size, name=name) for name in self.NORM_NAMES)

    def parts(self):
        return (self.mixer, self.feed_forward, self.norm_in, self.norm_post_mixer, self.norm_pre_ff,
                self.norm_post_ff)

    def param_specs(self, prefix: str) -> list[ParamSpec]:
        return [s for part in self.parts() for s in part.param_specs(prefix)]

    def bind(self, tensors, prefix, device, dtype) -> None:
        for part in self.parts():
            part.bind(tensors, prefix, device, dtype)

    def entry_norm(self) -> Optional[Norm]:
        return self.norm_in

    def forward(self, x: torch.Tensor, step, cache, entered: Optional[torch.Tensor] = None,
                then: Optional[Norm] = None) -> Optional[torch.Tensor]:
        h = entered if entered is not None else self.norm_in.forward(x)
        a = self.mixer.forward(h, step, cache)
        h = self.norm_post_mixer.add_into(a, x, then=self.norm_pre_ff)
        f = self.feed_forward.forward(h, step)
        return self.norm_post_ff.add_into(f, x, then=then)


BLOCKS.register("sandwich", SandwichBlock)
