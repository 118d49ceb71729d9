"""Arrangements of a layer's parts around the residual stream."""

from __future__ import annotations

from .base import Block, LayerCache, Part, PartSpec
from .registry import build_part
from .residual import ResidualStream


class PreNormBlock(Block):
    """h += mixer(norm1(h)); h += feed_forward(norm2(h)).

    Reference: somi_inference/models/qwen2.py:325-339.  ``names`` gives the
    sub-prefixes of the four parts under the layer's prefix.
    """
    graph_safe = True

    DEFAULT_NAMES = {"mixer_norm": "input_layernorm", "mixer": "self_attn",
                     "ffn_norm": "post_attention_layernorm", "feed_forward": "mlp"}

    def __init__(self, prefix: str, mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec,
                 ffn_norm: PartSpec, names: dict[str, str] | None = None) -> None:
        super().__init__(prefix)
        sub = dict(self.DEFAULT_NAMES)
        sub.update(names or {})
        self.mixer_norm = build_part("norm", mixer_norm, prefix=self.name(sub["mixer_norm"]))
        self.mixer = build_part("mixer", mixer, prefix=self.name(sub["mixer"]))
        self.ffn_norm = build_part("norm", ffn_norm, prefix=self.name(sub["ffn_norm"]))
        self.feed_forward = build_part("feed_forward", feed_forward, prefix=self.name(sub["feed_forward"]))

    def parts(self) -> list[Part]:
        return [self.mixer_norm, self.mixer, self.ffn_norm, self.feed_forward]

    def forward(self, stream: ResidualStream, step, cache: LayerCache | None) -> None:
        x = stream.normed(self.mixer_norm, lazy=getattr(self.mixer, "takes_normed_rows", False))
        stream.add(self.mixer.forward(x, step, cache))
        x = stream.normed(self.ffn_norm, lazy=getattr(self.feed_forward, "takes_normed_rows", False))
        stream.add(self.feed_forward.forward(x, step))
