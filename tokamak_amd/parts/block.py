"""Arrangements of a layer's parts."""

from __future__ import annotations

from tokamak_amd.config.registry import register_part
from tokamak_amd.kernels.linear import Added, StreamSink
from tokamak_amd.parts.base import Block, BranchPair
from tokamak_amd.parts.scale import scaled_sum


class PreNormBlock(Block):
    """x = x + mixer(norm(x)); x = x + feed_forward(norm(x))
    (reference: src/tokamak/model/transformer.py:107-108).

    The residual stream ``resid`` is float32.  Each sub-layer's output is left
    ``pending`` and added by the next norm's fused kernel, so the sum is formed
    in float32 and the stream is written once per sub-layer.  Parts that can
    (``fuses_residual``) are offered the stream itself, so that in a decode step
    of few rows their last product adds into it and the next product finishes
    the norm, with no kernel in between.  An optional ``position`` part prepares
    the step's position data for the mixer.  The feed-forward and its norm may be
    absent together: the layer is then x = x + mixer(norm(x)) alone.
    """

    roles = ("mixer_norm", "mixer")
    optional = ("position", "feed_forward_norm", "feed_forward")
    fuses_residual = True
    replays_parts = True

    def __init__(self, parts) -> None:
        super().__init__(parts)
        self.mixer_norm = parts["mixer_norm"]
        self.feed_forward_norm = parts.get("feed_forward_norm")
        self.feed_forward = parts.get("feed_forward")
        if (self.feed_forward is None) != (self.feed_forward_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.position = parts.get("position")
        self.entry_norm = self.mixer_norm

    def forward(self, resid, pending, batch, store, writes_cache, then=None):
        position = None if self.position is None else self.position.prepare(batch)
        h = _normed(self.mixer_norm, resid, pending, self.mixer)
        if self.feed_forward is None:
            return self.mixer.forward(h, batch, store, writes_cache, position, **_sink(self.mixer, then, resid))
        into = _sink(self.mixer, self.feed_forward_norm, resid)
        pending = self.mixer.forward(h, batch, store, writes_cache, position, **into)
        h = _normed(self.feed_forward_norm, resid, pending, self.feed_forward)
        into = _sink(self.feed_forward, then, resid)
        return _whole(self.feed_forward.forward(h, batch, **into))


def _whole(out):
    """A feed-forward's output as one pending sub-layer output (its terms, if it has several, as a pair)."""
    return BranchPair(*out) if isinstance(out, tuple) else out


def _normed(norm, resid, pending, consumer):
    """norm(resid + pending) for ``consumer``; left for the consumer to finish if both know how."""
    if norm.fuses_residual:
        return norm.forward(resid, pending, defer=consumer.fuses_residual)
    return norm.forward(resid, None if isinstance(pending, Added) else pending)


def _sink(producer, next_norm, resid) -> dict:
    """The keyword with which ``producer`` is offered the stream, if it can use it."""
    if not producer.fuses_residual:
        return {}
    if next_norm is not None and next_norm.fuses_residual:
        return {"add_into": next_norm.sink(resid)}
    return {"add_into": StreamSink(resid, None)}


class ParallelMixersBlock(Block):
    """x = x + scale_1 * (left_weight * left(norm(x)) + right_weight * right(norm(x)));
    x = x + scale_2 * feed_forward(norm(x)).

    Two mixers side by side read the same normed input, each with a cache slot of its own.
    ``mixer_scale`` and ``feed_forward_scale`` are per-coordinate layer scales (absent: ones);
    the feed-forward with its norm and scale may be absent altogether.  The weighted sum and
    the layer scale are formed in float32 from the branches' products, and the norm that reads
    the stream next adds the result into it.
    """

    roles = ("mixer_norm", "left", "right")
    optional = ("mixer_scale", "feed_forward_norm", "feed_forward", "feed_forward_scale")
    replays_parts = True

    def __init__(self, parts, *, left_weight: float = 1.0, right_weight: float = 1.0) -> None:
        super().__init__(parts)
        self.left_weight, self.right_weight = float(left_weight), float(right_weight)
        self.mixer_norm, self.left, self.right = parts["mixer_norm"], parts["left"], parts["right"]
        self.mixer_scale = parts.get("mixer_scale")
        self.feed_forward = parts.get("feed_forward")
        self.feed_forward_norm = parts.get("feed_forward_norm")
        self.feed_forward_scale = parts.get("feed_forward_scale")
        if (self.feed_forward is None) != (self.feed_forward_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        if self.feed_forward is None and self.feed_forward_scale is not None:
            raise ValueError("a feed-forward scale without a feed-forward")
        self.entry_norm = self.mixer_norm

    def forward(self, resid, pending, batch, store, writes_cache):
        h = self.mixer_norm.forward(resid, pending)
        left = self.left.forward(h, batch, store["left"], writes_cache, None)
        right = self.right.forward(h, batch, store["right"], writes_cache, None)
        dim, dtype = resid.shape[1], h.dtype
        weight = None if self.mixer_scale is None else self.mixer_scale.weight
        pending = scaled_sum(left, self.left_weight, right, self.right_weight, weight, dim, dtype)
        if self.feed_forward is None:
            return pending
        h = self.feed_forward_norm.forward(resid, pending)
        out = self.feed_forward.forward(h, batch)
        if self.feed_forward_scale is None:
            return out
        return scaled_sum(out, 1.0, None, 0.0, self.feed_forward_scale.weight, dim, dtype)


class ParallelSublayersBlock(Block):
    """h = norm(x); x = x + branch_scale * (mixer(h) + feed_forward(h)).

    The mixer and the feed-forward read the same stream, and their outputs are added to each other
    first and to the residual stream once, in float32, by the norm that reads the stream next (it
    receives them as a ``BranchPair``).  With a ``feed_forward_norm`` the feed-forward has a norm of
    its own over the same x: x = x + branch_scale * (mixer(norm(x)) + feed_forward(feed_forward_norm(x)));
    where the two norms agree on everything but their weights one kernel makes both outputs.  The
    feed-forward may be absent: x = x + branch_scale * mixer(h).  A feed-forward may return two terms
    (routed and shared experts) and leave a bias of its last product to the add (``output_bias``).
    An optional ``position`` part prepares the step's position data for the mixer.
    """

    roles = ("norm", "mixer")
    optional = ("position", "feed_forward", "feed_forward_norm")
    replays_parts = True

    def __init__(self, parts, *, branch_scale: float = 1.0) -> None:
        super().__init__(parts)
        self.branch_scale = float(branch_scale)
        self.norm = parts["norm"]
        self.feed_forward = parts.get("feed_forward")
        self.feed_forward_norm = parts.get("feed_forward_norm")
        if self.feed_forward_norm is not None and self.feed_forward is None:
            raise ValueError("a feed-forward norm without a feed-forward")
        self.position = parts.get("position")
        self.entry_norm = self.norm

    def _normed(self, resid, pending):
        """(the mixer's input, the feed-forward's)."""
        if self.feed_forward_norm is None:
            h = self.norm.forward(resid, pending)
            return h, h
        pair = getattr(self.norm, "forward_pair", None)
        both = pair(self.feed_forward_norm, resid, pending) if pair is not None else None
        if both is not None:
            return both
        h = self.norm.forward(resid, pending)
        return h, self.feed_forward_norm.forward(resid, None)

    def forward(self, resid, pending, batch, store, writes_cache):
        position = None if self.position is None else self.position.prepare(batch)
        h, h_ff = self._normed(resid, pending)
        mixed = self.mixer.forward(h, batch, store, writes_cache, position)
        if self.feed_forward is None:
            return mixed if self.branch_scale == 1.0 else BranchPair(mixed, scale=self.branch_scale)
        bias = getattr(self.feed_forward, "output_bias", None)
        out = self.feed_forward.forward(h_ff, batch, defer_bias=True) if bias is not None else self.feed_forward.forward(h_ff, batch)
        terms = out if isinstance(out, tuple) else (out,)
        if len(terms) > 2:
            raise ValueError("a feed-forward hands on two terms at most")
        return BranchPair(mixed, *terms, bias=bias, scale=self.branch_scale)


register_part("block", "pre_norm", PreNormBlock)
register_part("block", "parallel_sublayers", ParallelSublayersBlock)
register_part("block", "parallel_mixers", ParallelMixersBlock)
