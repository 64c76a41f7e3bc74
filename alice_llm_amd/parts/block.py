"""Block arrangements: how a layer's mixer, feed-forward and norms are wired to the residual stream.

"sandwich": x += post_mixer(mixer(pre_mixer(x))); x += post_ff(ff(pre_ff(x))), each norm optional
(llama3.rs:14178, 14460-14470, 14497, 14543-14557: Gemma 2 has all four; a pre-norm-only layer
leaves the post norms out and is the same wiring).
"""
from __future__ import annotations

from typing import Dict

from .base import BLOCKS


@BLOCKS.register("sandwich")
class SandwichBlock:
    graph_safe = True

    def __init__(self, mixer, feed_forward, norms: Dict[str, object]):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms

    def forward(self, stream, ctx, cache) -> None:
        # In decode steps parts that say so take their input in the matrix-core kernels' fragment order.
        frag = getattr(ctx, "fragment_activations", False)
        h = stream.normed(self.norms.get("pre_mixer"),
                          fragments=frag and getattr(self.mixer, "accepts_fragment_activations", False))
        stream.push(self.mixer.forward(h, ctx, cache), self.norms.get("post_mixer"))
        h = stream.normed(self.norms.get("pre_ff"),
                          fragments=frag and getattr(self.feed_forward, "accepts_fragment_activations", False))
        stream.push(self.feed_forward.forward(h, ctx), self.norms.get("post_ff"))


BLOCKS.register("prenorm", SandwichBlock)
