"""Arrangements of parts in a block.

An arrangement says which named parts it is made of and what each is (``roles``: name ->
``"norm"``, ``"mixer"`` or ``"feed_forward"``, the registry its kind is looked up in), and in
which order they run; ``mixer`` is the part whose ``cache_spec`` decides what the block's cache
entry holds.  The model builds the parts that the block's spec names and hands them
over as a dict; an arrangement with another number of parts declares other roles."""

import torch

from ..ops import kernels
from .registry import register_arrangement


@register_arrangement("pre_norm")
class PreNormBlock:
    """``h += mixer(norm1(h))`` then ``h += feed_forward(norm2(h))``
    (src/model/paged_decoder.py:181-189,210-228)."""

    roles = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "feed_forward": "feed_forward"}

    def __init__(self, width, dtype, parts):
        self.width = width
        self.dtype = dtype
        self._parts = dict(parts)
        self.norm1 = parts["norm1"]
        self.mixer = parts["mixer"]
        self.norm2 = parts["norm2"]
        self.feed_forward = parts["feed_forward"]

    @property
    def graph_safe(self):
        """The arrangement itself looks at no host value of the step; its parts decide."""
        return all(getattr(part, "graph_safe", False) for part in self.parts().values())

    def parts(self):
        return dict(self._parts)

    def _normed(self, norm, part, h, ctx):
        """Input of ``part``: the norm as a pending object if the part takes one, else rows."""
        scratch = ctx.workspace.first_rows("normed", self.width, self.dtype, ctx.tokens)
        if getattr(part, "accepts_pending_norm", False):
            pending = norm.pending(h, scratch)
            if pending is not None:
                return pending
        return norm.forward(h, scratch)

    def forward(self, h, ctx, cache):
        self.mixer.forward(self._normed(self.norm1, self.mixer, h, ctx), h, ctx, cache)
        self.feed_forward.forward(self._normed(self.norm2, self.feed_forward, h, ctx), h, ctx)
        return h


@register_arrangement("pre_norm_mixer")
class PreNormMixerBlock(PreNormBlock):
    """``h += mixer(norm1(h))`` alone: a layer without a feed-forward."""

    roles = {"norm1": "norm", "mixer": "mixer"}

    def __init__(self, width, dtype, parts):
        self.width = width
        self.dtype = dtype
        self._parts = dict(parts)
        self.norm1 = parts["norm1"]
        self.mixer = parts["mixer"]

    def forward(self, h, ctx, cache):
        self.mixer.forward(self._normed(self.norm1, self.mixer, h, ctx), h, ctx, cache)
        return h


_STREAM_WRITE = "stream_write"   # key of ``ctx.extra``: a sublayer's result that is not written back yet


@register_arrangement("hyper_connected")
class HyperConnectedBlock:
    """A pre-norm layer over a residual stream of several copies (``h`` is ``[T, streams *
    width]``): each sublayer reads a weighted sum of the copies through its norm and its result
    is mixed back into all of them (``parts/connection.py``).  Writing a result back and
    reading for the next sublayer is one launch; the last write of a block is left to the next
    block's first launch (``ctx.extra``), or to ``finish``."""

    roles = {"connect1": "connection", "norm1": "norm", "mixer": "mixer",
             "connect2": "connection", "norm2": "norm", "feed_forward": "feed_forward"}
    takes_stream_write = True

    def __init__(self, width, dtype, parts):
        self.width = width
        self.dtype = dtype
        self._parts = dict(parts)
        self.mixer = parts["mixer"]
        self.sublayers = [(parts["connect1"], parts["norm1"], self.mixer)]
        if "feed_forward" in parts:
            self.sublayers.append((parts["connect2"], parts["norm2"], parts["feed_forward"]))
        self.streams = parts["connect1"].streams

    @property
    def graph_safe(self):
        return all(getattr(part, "graph_safe", False) for part in self._parts.values())

    def parts(self):
        return dict(self._parts)

    def forward(self, h, ctx, cache):
        tokens = ctx.tokens
        normed = ctx.workspace.first_rows("normed", self.width, self.dtype, tokens)
        # the sublayers' last products add into y, which every launch below leaves cleared
        y = ctx.workspace.first_rows("sublayer", self.width, torch.float32, tokens)
        if ctx.extra is None:
            ctx.extra = {}
        write = ctx.extra.pop(_STREAM_WRITE, None)
        for connection, norm, part in self.sublayers:
            kernels.hyper_step(h, tokens, self.width, self.streams, write=write,
                               read=connection.read_of(norm, normed), zero=y)
            if part is self.mixer:
                part.forward(normed, y, ctx, cache)
            else:
                part.forward(normed, y, ctx)
            write = connection.write_of(y)
        ctx.extra[_STREAM_WRITE] = write
        return h

    def finish(self, h, ctx):
        """Write back what the last sublayer left (no block follows that would)."""
        write = ctx.extra.pop(_STREAM_WRITE, None) if ctx.extra else None
        if write is not None:
            kernels.hyper_step(h, ctx.tokens, self.width, self.streams, write=write)


@register_arrangement("hyper_connected_mixer")
class HyperConnectedMixerBlock(HyperConnectedBlock):
    """The same with a mixer only."""

    roles = {"connect1": "connection", "norm1": "norm", "mixer": "mixer"}


_SCALED_ADD = "scaled_add"    # key of ``ctx.extra``: (y, factor) of a block that is not added to the stream yet
STREAM_BIAS = "stream_bias"   # key of ``ctx.extra``: a float row that the next block adds to every token


@register_arrangement("parallel_scaled")
class ParallelScaledBlock:
    """``h += factor * (mixer(u) + feed_forward(u))`` with ``u = norm1(h)``: one norm, both
    sublayers read its output.  The sublayers add into a float row ``y`` per token, which one
    launch folds into the stream; that launch is the next block's first, which also adds the row
    that the model puts before a pass (``ctx.extra[STREAM_BIAS]``), norms for the next block and
    clears ``y`` (``kernels.stream_step``).  ``finish`` writes back where no such block follows."""

    roles = {"norm1": "norm", "mixer": "mixer", "feed_forward": "feed_forward"}
    takes_stream_write = True
    takes_stream_bias = True

    def __init__(self, width, dtype, parts, factor: float = 1.0):
        self.width = width
        self.dtype = dtype
        self.factor = float(factor)
        self._parts = dict(parts)
        self.norm1 = parts["norm1"]
        self.mixer = parts["mixer"]
        self.feed_forward = parts.get("feed_forward")
        if not hasattr(self.norm1, "gamma_eps"):
            raise ValueError("a parallel block needs an RMS norm without a shift")

    @property
    def graph_safe(self):
        return all(getattr(part, "graph_safe", False) for part in self._parts.values())

    def parts(self):
        return dict(self._parts)

    def forward(self, h, ctx, cache):
        tokens = ctx.tokens
        normed = ctx.workspace.first_rows("normed", self.width, self.dtype, tokens)
        # (made cleared; every launch that folds it into the stream clears it again)
        ctx.workspace.rows("sublayer_sum", self.width, torch.float32, cleared=True)
        y = ctx.workspace.first_rows("sublayer_sum", self.width, torch.float32, tokens)
        if ctx.extra is None:
            ctx.extra = {}
        gamma, eps = self.norm1.gamma_eps()
        add = ctx.extra.pop(_SCALED_ADD, None)
        kernels.stream_step(h, tokens, self.width, add=add, bias=ctx.extra.pop(STREAM_BIAS, None),
                            norm=(gamma, eps, normed), zero=None if add is None else add[0])
        self.mixer.forward(normed, y, ctx, cache)
        if self.feed_forward is not None:
            self.feed_forward.forward(normed, y, ctx)
        ctx.extra[_SCALED_ADD] = (y, self.factor)
        return h

    def finish(self, h, ctx):
        """Fold in what the block left (no block follows that would)."""
        add = ctx.extra.pop(_SCALED_ADD, None) if ctx.extra else None
        if add is not None:
            kernels.stream_step(h, ctx.tokens, self.width, add=add, zero=add[0])


@register_arrangement("pre_norm_scaled")
class PreNormScaledBlock:
    """``h += scale1 * mixer(norm1(h))`` then ``h += scale2 * feed_forward(norm2(h))`` with a
    learned factor per column on each sublayer's result (``parts/connection.py: column_scale``).
    A sublayer adds into a float row ``y`` per token; one launch folds ``scale * y`` of the
    sublayer before into the stream, norms for the next one and clears ``y``
    (``kernels.stream_step``).  A block's last sum is left to the next block's first launch, or
    to ``finish``."""

    roles = {"norm1": "norm", "mixer": "mixer", "scale1": "connection",
             "norm2": "norm", "feed_forward": "feed_forward", "scale2": "connection"}
    takes_stream_write = True

    def __init__(self, width, dtype, parts):
        self.width = width
        self.dtype = dtype
        self._parts = dict(parts)
        self.mixer = parts["mixer"]
        self.sublayers = [(parts["norm1"], self.mixer, parts["scale1"])]
        if "feed_forward" in parts:
            self.sublayers.append((parts["norm2"], parts["feed_forward"], parts["scale2"]))
        for norm, _, _ in self.sublayers:
            if not hasattr(norm, "gamma_eps"):
                raise ValueError("a scaled pre-norm block needs RMS norms without a shift")

    @property
    def graph_safe(self):
        return all(getattr(part, "graph_safe", False) for part in self._parts.values())

    def parts(self):
        return dict(self._parts)

    def forward(self, h, ctx, cache):
        tokens = ctx.tokens
        normed = ctx.workspace.first_rows("normed", self.width, self.dtype, tokens)
        # (made cleared; every launch that folds it into the stream clears it again)
        ctx.workspace.rows("sublayer_sum", self.width, torch.float32, cleared=True)
        y = ctx.workspace.first_rows("sublayer_sum", self.width, torch.float32, tokens)
        if ctx.extra is None:
            ctx.extra = {}
        add = ctx.extra.pop(_SCALED_ADD, None)
        for norm, part, scale in self.sublayers:
            gamma, eps = norm.gamma_eps()
            kernels.stream_step(h, tokens, self.width, add=add, norm=(gamma, eps, normed),
                                zero=None if add is None else add[0])
            if part is self.mixer:
                part.forward(normed, y, ctx, cache)
            else:
                part.forward(normed, y, ctx)
            add = (y, 1.0, scale.weight)
        ctx.extra[_SCALED_ADD] = add
        return h

    def finish(self, h, ctx):
        """Fold in what the block left (no block follows that would)."""
        add = ctx.extra.pop(_SCALED_ADD, None) if ctx.extra else None
        if add is not None:
            kernels.stream_step(h, ctx.tokens, self.width, add=add, zero=add[0])


@register_arrangement("pre_norm_scaled_mixer")
class PreNormScaledMixerBlock(PreNormScaledBlock):
    """The same with a mixer only."""

    roles = {"norm1": "norm", "mixer": "mixer", "scale1": "connection"}


@register_arrangement("parallel_scaled_mixer")
class ParallelScaledMixerBlock(ParallelScaledBlock):
    """The same with a mixer only."""

    roles = {"norm1": "norm", "mixer": "mixer"}
