"""Block arrangements: how a layer's mixer, feed-forward and norms are wired to the residual stream.

"sandwich": x += post_mixer(mixer(pre_mixer(x))); x += post_ff(ff(pre_ff(x))), each norm optional
(llama3.rs:14178, 14460-14470, 14497, 14543-14557: Gemma 2 has all four; a pre-norm-only layer
leaves the post norms out and is the same wiring).  The feed-forward may be absent, and a mixer may return
several branches, each with a post norm of its own, which are all added before the feed-forward's norm.

"parallel": one norm, whose output feeds the mixer and the feed-forward side by side:
h = pre(x); x += mixer(h) + ff(h) (the feed-forward may be absent); then the layer's extras act on the
stream in their order (a per-layer token input, say).  A mixer may return several branches, each with a post
norm of its own.
"""
from __future__ import annotations

from typing import Dict

from .base import BLOCKS


@BLOCKS.register("sandwich")
class SandwichBlock:
    graph_safe = True

    def __init__(self, mixer, feed_forward, norms: Dict[str, object], extras: Dict[str, object] = None):
        if extras:
            raise ValueError("the sandwich arrangement has no place for further parts of a layer")
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms

    def forward(self, stream, ctx, cache) -> None:
        # In decode steps parts that say so take their input in the matrix-core kernels' fragment order.
        frag = getattr(ctx, "fragment_activations", False)
        h = stream.normed(self.norms.get("pre_mixer"),
                          fragments=frag and getattr(self.mixer, "accepts_fragment_activations", False))
        branches = self.mixer.forward(h, ctx, cache)
        if isinstance(branches, list):
            stream.push_many([(b, post if post is not None else self.norms.get("post_mixer")) for b, post in branches])
        else:
            stream.push(branches, self.norms.get("post_mixer"))
        if self.feed_forward is None:
            return
        h = stream.normed(self.norms.get("pre_ff"),
                          fragments=frag and getattr(self.feed_forward, "accepts_fragment_activations", False))
        stream.push(self.feed_forward.forward(h, ctx), self.norms.get("post_ff"))


BLOCKS.register("prenorm", SandwichBlock)


@BLOCKS.register("parallel")
class ParallelBlock:
    def __init__(self, mixer, feed_forward, norms: Dict[str, object], extras: Dict[str, object] = None):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.norms = norms
        self.extras = dict(extras or {})

    @property
    def graph_safe(self) -> bool:
        return True

    def forward(self, stream, ctx, cache) -> None:
        h = stream.normed(self.norms.get("pre"))
        branches = self.mixer.forward(h, ctx, cache)
        if not isinstance(branches, list):
            branches = [(branches, None)]
        if self.feed_forward is not None:
            branches.append((self.feed_forward.forward(h, ctx), None))
        stream.push_many(branches)                              # one kernel adds them all
        for extra in self.extras.values():
            extra.forward(stream, ctx)
