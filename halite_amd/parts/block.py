"""How the parts of a layer are arranged (src/halite/transformers/block.py:10-85).

An arrangement says which parts it is made of, by name and by kind of part
(``roles``), which of them may be left out (``optional``), and how a step's tokens
go through them.  The builder makes the parts that the layer's description names,
refuses names that the arrangement does not have, and hands the arrangement a dict.
One part of every arrangement is its ``mixer``: the part that may own a cache and
per-request state, which the step function binds to every run of the layer.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import CONNECTIONS, FEED_FORWARDS, MIXERS, NORMS, Arrangement, register_arrangement
from .norm import RMSNorm


@register_arrangement("pre_norm")
class PreNormBlock(Arrangement):
    """``h = h + mixer(norm(h)); h = h + ff(norm(h))`` (block.py:56-74).

    The residual stream ``h`` is float32.  Each add is done by the norm that
    follows it, so the block hands its last delta on to the next block's first
    norm (or to the model's final norm) instead of adding it itself.
    """

    graph_safe = True
    roles = {"mixer_norm": NORMS, "mixer": MIXERS, "ff_norm": NORMS, "ff": FEED_FORWARDS}
    takes_next_norm = True  # forward() accepts next_norm=

    def __init__(self, parts):
        super().__init__(parts)
        self.mixer_norm, self.ff_norm, self.ff = parts["mixer_norm"], parts["ff_norm"], parts["ff"]

    # The norm between two parts can be folded into the products around it where the part
    # before it offers that and the part after it takes such rows.
    def first_norm_for(self, h):
        """For the block that runs before this one: what its last product may prepare."""
        return self.mixer_norm.foldable(h) if self.mixer.takes_normed_rows else None

    def forward(self, h, pending, ctx, run, next_norm=None):
        x = self.mixer_norm.forward(h, delta=pending)
        then = None
        if self.mixer.folds_next_norm and self.ff.takes_normed_rows:
            then = self.ff_norm.foldable(h)
        a = self.mixer.forward(x, ctx, run, then=then) if then is not None else self.mixer.forward(x, ctx, run)
        x = self.ff_norm.forward(h, delta=a)
        if next_norm is not None and self.ff.folds_next_norm:
            return self.ff.forward(x, ctx, then=next_norm)
        return self.ff.forward(x, ctx)


@register_arrangement("parallel")
class ParallelBlock(Arrangement):
    """``h = h + (mixer(norm_a(h)) + ff(norm_b(h)))``: the mixer and the feed-forward read
    the same rows of the stream, each through a norm of its own; a layer may leave the
    feed-forward (and its norm) out.

    Both parts are handed the float32 stream to add their result into (``add_to``), so
    the sum is float32 and nothing is left pending.  Where both norms are RMSNorms of one
    eps in the unrounded order, one kernel computes the statistic once and writes both
    results."""

    graph_safe = True
    roles = {"mixer_norm": NORMS, "mixer": MIXERS, "ff_norm": NORMS, "ff": FEED_FORWARDS}
    optional = ("ff_norm", "ff")

    def __init__(self, parts):
        super().__init__(parts)
        self.mixer_norm, self.ff_norm, self.ff = parts["mixer_norm"], parts.get("ff_norm"), parts.get("ff")
        if (self.ff is None) != (self.ff_norm is None):
            raise ValueError("a parallel block has a feed-forward and its norm, or neither")
        for name, part in (("mixer", self.mixer), ("ff", self.ff)):
            if part is not None and not getattr(part, "adds_to_stream", False):
                raise ValueError(f"a parallel block needs parts that add into the stream; {name} ({type(part).__name__}) does not")
        a, b = self.mixer_norm, self.ff_norm
        self._one_pass = (
            isinstance(a, RMSNorm) and isinstance(b, RMSNorm) and a.p.eps == b.p.eps
            and not a.p.round_before_weight and not b.p.round_before_weight
        )

    def forward(self, h, pending, ctx, run):
        if pending is not None:
            ops.residual_add(h, pending)
        if self.ff is None:
            x = self.mixer_norm.forward(h)
            self.mixer.forward(x, ctx, run, add_to=h)
            return None
        if self._one_pass and self.mixer_norm.weight.dtype == self.ff_norm.weight.dtype:
            x, y = ops.rmsnorm_exact(h, self.mixer_norm.weight, self.mixer_norm.p.eps, self.mixer_norm.build.dtype,
                                     second=self.ff_norm.weight)
        else:
            x, y = self.mixer_norm.forward(h), self.ff_norm.forward(h)
        # both results are computed before either is added: both parts read the same stream
        self.mixer.forward(x, ctx, run, add_to=h)
        self.ff.forward(y, ctx, add_to=h)
        return None


@register_arrangement("post_norm")
class PostNormBlock(Arrangement):
    """``h = h + norm_a(mixer(h)); h = h + norm_b(ff(h))``: the parts read the stream itself
    and the norm is on what they return.  A layer may leave the feed-forward (and its
    norm) out, and may close with a third part of the feed-forward kind, ``side``, with a norm
    of its own: ``h = h + norm_c(side(h))``.  A norm with a layer scale multiplies by its
    weight times that scale (``RMSNorm.multiplier``).

    The parts return float32 rows; norm, weight and sum are one float32 pass
    (``ops.post_norm_add``), which also leaves the new rows rounded to the activation type
    for the part that reads them next."""

    graph_safe = True
    roles = {"mixer": MIXERS, "mixer_norm": NORMS, "ff": FEED_FORWARDS, "ff_norm": NORMS,
             "side": FEED_FORWARDS, "side_norm": NORMS}
    optional = ("ff", "ff_norm", "side", "side_norm")

    def __init__(self, parts):
        super().__init__(parts)
        self.mixer_norm, self.ff_norm, self.ff = parts["mixer_norm"], parts.get("ff_norm"), parts.get("ff")
        # a third part of the feed-forward kind that closes the layer the same way:
        # h = h + norm_c(side(h))
        self.side, self.side_norm = parts.get("side"), parts.get("side_norm")
        if (self.ff is None) != (self.ff_norm is None) or (self.side is None) != (self.side_norm is None):
            raise ValueError("a post-norm block has a feed-forward (a side part) and its norm, or neither")
        for norm in (self.mixer_norm, self.ff_norm, self.side_norm):
            if norm is not None and not isinstance(norm, RMSNorm):
                raise ValueError(f"a post-norm block norms with RMSNorm; {type(norm).__name__} is another")

    def forward(self, h, pending, ctx, run):
        if pending is not None:
            ops.residual_add(h, pending)
        dtype = self.mixer.build.dtype
        # the rows as the block of the run before left them rounded, if that was one of this
        # kind (then nothing has touched the stream since)
        left = getattr(ctx, "rounded_rows", None)
        ctx.rounded_rows = None
        if pending is None and left is not None and left[0] == run.index - 1 and left[1].dtype == dtype and left[1].shape == h.shape:
            x = left[1]
        else:
            x = ops.cast_rows(h, dtype)
        norm = self.mixer_norm
        weight_of = lambda nm: getattr(nm, "multiplier", nm.weight)  # noqa: E731
        # a sum of two mixers is made by the kernel that norms it
        terms = self.mixer.forward_terms(x, ctx, run) if hasattr(self.mixer, "forward_terms") else None
        if terms is not None and len(terms) == 2:
            (a, s1), (b, s2) = terms
            x = ops.post_norm_add(h, a, weight_of(norm), norm.p.eps, cast_to=dtype, scale=s1, second=b, second_scale=s2)
        else:
            a = self.mixer.forward(x, ctx, run) if terms is None else None
            if terms is not None:  # any other number of members: added up one by one
                a = ops.scale_(terms[0][0], terms[0][1])
                for b, s in terms[1:]:
                    ops.scaled_sum_(a, 1.0, b, s)
            if a.dtype != torch.float32:
                a = a.float()
            x = ops.post_norm_add(h, a, weight_of(norm), norm.p.eps, cast_to=dtype)
        for part, part_norm in ((self.ff, self.ff_norm), (self.side, self.side_norm)):
            if part is None:
                continue
            b = part.forward(x, ctx)
            if b.dtype != torch.float32:
                b = b.float()
            x = ops.post_norm_add(h, b, weight_of(part_norm), part_norm.p.eps, cast_to=dtype)
        if dtype != torch.float32:
            ctx.rounded_rows = (run.index, x)
        return None


@register_arrangement("hyper_pre_norm")
class HyperPreNormBlock(Arrangement):
    """A pre-norm block on a residual stream that is kept in copies: each of the two parts
    reads its input through a connection of its own (``mixer_link``, ``ff_link``), which also
    says how the part's result gets back into the copies.  A layer may leave the
    feed-forward (with its norm and connection) out.

    The stream handed from block to block is ``[copies, T, width]`` float32.  A part's
    result is left pending, with its connection, for whoever reads next: the write of one
    part and the read and norm of the next are one pass over the copies."""

    graph_safe = True
    roles = {"mixer_norm": NORMS, "mixer": MIXERS, "mixer_link": CONNECTIONS,
             "ff_norm": NORMS, "ff": FEED_FORWARDS, "ff_link": CONNECTIONS}
    optional = ("ff_norm", "ff", "ff_link")

    def __init__(self, parts):
        super().__init__(parts)
        self.mixer_norm, self.mixer_link = parts["mixer_norm"], parts["mixer_link"]
        self.ff_norm, self.ff, self.ff_link = parts.get("ff_norm"), parts.get("ff"), parts.get("ff_link")
        if len({self.ff is None, self.ff_norm is None, self.ff_link is None}) != 1:
            raise ValueError("a block has a feed-forward with its norm and connection, or none of them")
        if self.ff_link is not None and self.ff_link.copies != self.mixer_link.copies:
            raise ValueError("a block's connections keep different numbers of copies")

    @property
    def stream_copies(self) -> int:
        return self.mixer_link.copies

    def forward(self, h, pending, ctx, run):
        x = self.mixer_link.step(h, pending, self.mixer_norm)
        pending = (self.mixer.forward(x, ctx, run), self.mixer_link)
        if self.ff is not None:
            x = self.ff_link.step(h, pending, self.ff_norm)
            pending = (self.ff.forward(x, ctx), self.ff_link)
        return pending

    def leave(self, h, pending, rows):
        """The model's one stream after the last block (of ``rows`` alone if given)."""
        link = pending[1] if pending is not None else self.mixer_link
        return link.leave(h, pending, rows)
