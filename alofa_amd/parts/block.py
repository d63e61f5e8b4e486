"""Arrangements of parts in a layer.

prenorm: a = hidden; a += mixer(norm0(a)); a += feed_forward(norm1(a)) — two
norms before their sub-layers, two residual sums in float32
(src/alofa/model/arch/qwen.mojo:1418-1510). It reads the layer's parts
``mixer``, ``feed_forward`` and ``norms`` (two).

scaled_prenorm: a += s0 * mixer(norm0(a)); a += s1 * feed_forward(norm1(a)), with s a vector per sub-layer (one factor per
channel, times a factor for all) and an optional feed-forward.

filtered_prenorm: the same as prenorm with a filter over time in front of every sub-layer, an optional feed-forward, and an
optional weighted average over the outputs of all layers so far.

sandwich: a += post0(mixer(pre0(a))); a += post1(feed_forward(pre1(a))): a norm in front of every sub-layer and one behind it, before
the sum; the feed-forward optional."""
from __future__ import annotations

import os

import torch

from .. import ops
from ..errors import AlofaError
from ..weights.loader import TensorRule
from .base import Block, build_part, register_part, tensors_of


class PreNormBlock(Block):
    n_norms = 2

    @classmethod
    def layer_tensors(cls, layer) -> dict:
        out = {}
        for n in layer.part("norms"):
            out.update(tensors_of("norm", n))
        out.update(tensors_of("mixer", layer.part("mixer")))
        out.update(tensors_of("feed_forward", layer.part("feed_forward")))
        return out

    def __init__(self, layer, weights, rt):
        super().__init__(layer, weights, rt)
        norms = layer.part("norms")
        if len(norms) != self.n_norms:
            raise AlofaError("invalid_argument", "a prenorm block takes two norms", f"prefix={layer.prefix} norms={len(norms)}")
        self.norms = [build_part("norm", n, weights, rt) for n in norms]
        self.mixer = build_part("mixer", layer.part("mixer"), weights, rt)
        self.feed_forward = build_part("feed_forward", layer.part("feed_forward"), weights, rt)
        self.parts = [*self.norms, self.mixer, self.feed_forward]

    def mixers(self):
        return [self.mixer]

    takes_normed = True

    def wants_normed(self, rows):
        return None if self.mixer.fuses_norm(self.norms[0], rows) else self.norms[0]

    def forward(self, ctx, entry, hidden, normed=None, then=None):
        """``normed``: the first norm's rows, where the block before has left them; ``then`` = (norm, rows): the norm
        the next block starts with, to be left in ``rows``. Returns whether that was done."""
        rows = hidden.shape[0]
        buf = ctx.scratch("normed", tuple(hidden.shape), self.rt.dtype)
        mixer, ff, (n0, n1) = self.mixer, self.feed_forward, self.norms
        # a norm rides on the first kernel of the part behind it where that can (a launch less where launches are what
        # a step costs); else the part before it sees to it, whose last launch may have whole rows in hand; else it
        # is a kernel of its own
        ff_rides = ff.fuses_norm(n1, rows)
        more = {"then": (n1, buf)} if not ff_rides and mixer.gives_normed and n1.as_rmsnorm() is not None else {}
        if normed is not None:
            mixer.forward(ctx, entry, normed, hidden, **more)
        elif mixer.fuses_norm(n0, rows):
            mixer.forward(ctx, entry, None, hidden, norm=n0, **more)
        else:
            n0.forward(buf, hidden)
            mixer.forward(ctx, entry, buf, hidden, **more)
        given = then is not None and ff.gives_normed
        more_ff = {"then": then} if given else {}
        if ff_rides:
            ff.forward(ctx, None, hidden, norm=n1, **more_ff)
        else:
            if not more:
                n1.forward(buf, hidden)
            ff.forward(ctx, buf, hidden, **more_ff)
        return given


class FilteredPreNormBlock(Block):
    """a += mixer(conv0(norm0(a))), then, where the layer has a feed-forward, a += feed_forward(conv1(norm1(a))): the
    rows every sub-layer reads pass a filter over time first (a part of the "conv" family that keeps its own state).
    Then, with ``depth_average`` (a tensor of as many weights as there are layer outputs so far, the embedding's
    counted), what goes on is the weighted sum of the outputs of all layers up to this one, each taken before its
    own averaging; the outputs live in a stack that the step keeps.

    It reads the layer's parts ``mixer``, ``norms`` and ``convs`` (one per sub-layer; a conv may be None) and
    ``feed_forward`` (may be None). params: depth_average (tensor name or None), level (this layer's place in
    the stack: it has level + 1 weights), levels (the stack's height), hidden."""

    @classmethod
    def layer_tensors(cls, layer) -> dict:
        out = {}
        for n in layer.part("norms"):
            out.update(tensors_of("norm", n))
        for c in layer.part("convs"):
            if c is not None:
                out.update(tensors_of("conv", c))
        out.update(tensors_of("mixer", layer.part("mixer")))
        if layer.part("feed_forward") is not None:
            out.update(tensors_of("feed_forward", layer.part("feed_forward")))
        if layer.block.get("depth_average") is not None:
            out[layer.block.params["depth_average"]] = TensorRule((layer.block.params["level"] + 1,), "average")
        return out

    def __init__(self, layer, weights, rt):
        super().__init__(layer, weights, rt)
        p = layer.block.params
        ff = layer.part("feed_forward")
        subs = 1 if ff is None else 2
        norms, convs = layer.part("norms"), layer.part("convs")
        if len(norms) != subs or len(convs) != subs:
            raise AlofaError("invalid_argument", "one norm and one filter (or None) per sub-layer", f"prefix={layer.prefix} sub-layers={subs} norms={len(norms)} convs={len(convs)}")
        self.norms = [build_part("norm", n, weights, rt) for n in norms]
        self.convs = [build_part("conv", c, weights, rt) if c is not None else None for c in convs]
        self.mixer = build_part("mixer", layer.part("mixer"), weights, rt)
        self.feed_forward = build_part("feed_forward", ff, weights, rt) if ff is not None else None
        self.level, self.levels = int(p.get("level", 0)), int(p.get("levels", 0))
        self.depth_weights = rt.vector(weights[p["depth_average"]]) if p.get("depth_average") is not None else None
        if self.depth_weights is not None and not 1 <= self.level < self.levels:
            raise AlofaError("invalid_argument", "a layer's level lies above the embedding's and within the stack", f"level={self.level} levels={self.levels}")
        self.parts = [p for p in (*self.norms, *self.convs, self.mixer, self.feed_forward) if p is not None]
        # the parts that keep a cache or state: the mixer's, then the filters
        self._stateful = [*self.mixer.stateful_parts(), *(c for c in self.convs if c is not None)]

    def mixers(self):
        return self._stateful

    def _read(self, ctx, entry, sub, hidden):
        """What sub-layer ``sub`` reads: its norm of the stream, filtered over time, in the activation dtype."""
        rows = ctx.scratch("normed", tuple(hidden.shape), self.rt.dtype)
        conv = self.convs[sub]
        if conv is None:
            self.norms[sub].forward(rows, hidden)
            return rows
        if conv.fuses_norm(ctx, self.norms[sub]):
            conv.forward(ctx, (entry, self._stateful.index(conv)), rows, hidden, norm=self.norms[sub])
            return rows
        wide = ctx.scratch("normed_f32", tuple(hidden.shape), torch.float32)
        self.norms[sub].forward(wide, hidden)
        conv.forward(ctx, (entry, self._stateful.index(conv)), rows, wide)
        return rows

    def forward(self, ctx, entry, hidden):
        stack = None
        if self.depth_weights is not None:
            stack = ctx.scratch("depth_stack", (self.levels, *hidden.shape), torch.float32)
            if self.level == 1:      # what the layers start from is the lowest level
                ops.depth_average(hidden, stack, None, 1, self.rt.exact)
        self.mixer.forward(ctx, (entry, 0), self._read(ctx, entry, 0, hidden), hidden)
        if self.feed_forward is not None:
            self.feed_forward.forward(ctx, self._read(ctx, entry, 1, hidden), hidden)
        if stack is not None:
            ops.depth_average(hidden, stack, self.depth_weights, self.level + 1, self.rt.exact)


class ScaledPreNormBlock(Block):
    """Pre-norm sub-layers whose results are multiplied channel by channel before they join the stream:
    a += r * ls0 * mixer(norm0(a)), then, where the layer has a feed-forward, a += r * ls1 * feed_forward(norm1(a)).
    It reads the layer's parts ``mixer``, ``norms`` (one per sub-layer) and ``feed_forward`` (may be None).
    params: hidden, residual_scale (r), channel_scales (tensor names, one per sub-layer, each [hidden]; a name may be None).
    A part that says ``takes_channel_scale`` is handed the vector (``scale=``) and applies it as it adds; any other part
    leaves its result apart (``out=``) and the block adds it."""

    @classmethod
    def layer_tensors(cls, layer) -> dict:
        out = {}
        for n in layer.part("norms"):
            out.update(tensors_of("norm", n))
        out.update(tensors_of("mixer", layer.part("mixer")))
        if layer.part("feed_forward") is not None:
            out.update(tensors_of("feed_forward", layer.part("feed_forward")))
        for name in layer.block.params["channel_scales"]:
            if name is not None:
                out[name] = TensorRule((layer.block.params["hidden"],), "norm")
        return out

    def __init__(self, layer, weights, rt):
        super().__init__(layer, weights, rt)
        p = layer.block.params
        ff = layer.part("feed_forward")
        subs = 1 if ff is None else 2
        norms, names = layer.part("norms"), p["channel_scales"]
        if len(norms) != subs or len(names) != subs:
            raise AlofaError("invalid_argument", "one norm and one channel scale (or None) per sub-layer", f"prefix={layer.prefix} sub-layers={subs} norms={len(norms)} scales={len(names)}")
        self.norms = [build_part("norm", n, weights, rt) for n in norms]
        self.mixer = build_part("mixer", layer.part("mixer"), weights, rt)
        self.feed_forward = build_part("feed_forward", ff, weights, rt) if ff is not None else None
        r, h = float(p.get("residual_scale", 1.0)), int(p["hidden"])
        # (the factor for all channels and the channels' own, multiplied once, in float64, and kept as float32)
        self.scales = [rt.vector(((weights[n].double() if n is not None else torch.ones(h, dtype=torch.float64)) * r).float()) for n in names]
        self.parts = [p for p in (*self.norms, self.mixer, self.feed_forward) if p is not None]

    def mixers(self):
        return self.mixer.stateful_parts()

    def _sub_layer(self, ctx, part, norm, scale, hidden, buf, where=(), normed=False, then=None):
        """hidden += scale * part(norm(hidden)). ``normed``: ``buf`` holds norm(hidden) already. ``then`` = (weight, eps, rows): the RMSNorm of
        the new stream is left in ``rows`` on the way. A norm rides on the part's first product where the part says it can."""
        rows = hidden.shape[0]
        if getattr(part, "takes_channel_scale", False):
            more = {"then": then} if then is not None else {}
            if not normed and part.fuses_norm(norm, rows):
                part.forward(ctx, *where, None, hidden, scale=scale, norm=norm, **more)
            else:
                if not normed:
                    norm.forward(buf, hidden)
                part.forward(ctx, *where, buf, hidden, scale=scale, **more)
            return
        if not normed:
            norm.forward(buf, hidden)
        apart = ctx.scratch("sub_out", tuple(hidden.shape), torch.float32)
        part.forward(ctx, *where, buf, hidden, out=apart)
        if then is None:
            ops.add_channel_scaled(hidden, apart, scale, self.rt.exact)
        else:
            ops.add_channel_scaled_norm(hidden, apart, scale, *then, exact=self.rt.exact)

    def forward(self, ctx, entry, hidden):
        buf = ctx.scratch("normed", tuple(hidden.shape), self.rt.dtype)
        ff = self.feed_forward
        then = None
        if ff is not None and FUSE_SUMS and self.norms[1].as_rmsnorm() is not None and not (getattr(ff, "takes_channel_scale", False) and ff.fuses_norm(self.norms[1], hidden.shape[0])):
            # the norm in front of the feed-forward is made by the launch that adds the mixer's result to the stream
            then = (*self.norms[1].as_rmsnorm(), buf)
        self._sub_layer(ctx, self.mixer, self.norms[0], self.scales[0], hidden, buf, where=((entry, 0),), then=then)
        if ff is not None:
            self._sub_layer(ctx, ff, self.norms[1], self.scales[1], hidden, buf, normed=then is not None)


class SandwichBlock(Block):
    """a += post0(mixer(pre0(a))), then, where the layer has a feed-forward, a += post1(feed_forward(pre1(a))).
    It reads the layer's parts ``mixer``, ``feed_forward`` (may be None) and ``norms``: (pre0, post0) or (pre0, post0, pre1, post1).
    Mixer and feed-forward leave their results apart (``out=``); a layer norm behind a sub-layer is applied by the launch that adds
    to the stream, any other norm runs where the result lies and a sum follows. Where the norm behind a sub-layer and the one in front of
    the next (the feed-forward's, or the next block's first) are both layer norms, one launch adds and leaves the next one's input."""

    @classmethod
    def layer_tensors(cls, layer) -> dict:
        out = {}
        for n in layer.part("norms"):
            out.update(tensors_of("norm", n))
        out.update(tensors_of("mixer", layer.part("mixer")))
        if layer.part("feed_forward") is not None:
            out.update(tensors_of("feed_forward", layer.part("feed_forward")))
        return out

    def __init__(self, layer, weights, rt):
        super().__init__(layer, weights, rt)
        ff = layer.part("feed_forward")
        norms = layer.part("norms")
        if len(norms) != (2 if ff is None else 4):
            raise AlofaError("invalid_argument", "a norm in front of and one behind every sub-layer", f"prefix={layer.prefix} norms={len(norms)} feed_forward={ff is not None}")
        self.norms = [build_part("norm", n, weights, rt) for n in norms]
        self.mixer = build_part("mixer", layer.part("mixer"), weights, rt)
        self.feed_forward = build_part("feed_forward", ff, weights, rt) if ff is not None else None
        self.parts = [p for p in (*self.norms, self.mixer, self.feed_forward) if p is not None]

    def mixers(self):
        return self.mixer.stateful_parts()

    def _join(self, hidden, apart, norm):
        ln = norm.as_layernorm()
        if ln is not None:
            ops.layernorm_add(hidden, apart, *ln, exact=self.rt.exact)
        else:
            norm.forward(apart, apart)
            ops.add_scaled(hidden, apart, 1.0, exact=self.rt.exact)

    takes_normed = True
    leaves_layernorm = True      # the launch that adds this block's last result can leave the next block's layer norm

    def wants_normed(self, rows):
        return self.norms[0]

    def _join_then(self, hidden, apart, norm, then) -> bool:
        """The sum behind ``norm`` into the stream; with ``then`` = (the norm the next reader starts with, rows) and both of them layer
        norms, the same launch leaves those rows. Returns whether it did."""
        behind = norm.as_layernorm()
        front = then[0].as_layernorm() if then is not None else None
        if behind is not None and front is not None and FUSE_SUMS:
            ops.layernorm_add_norm(hidden, apart, *behind, then[1], *front, exact=self.rt.exact)
            return True
        self._join(hidden, apart, norm)
        return False

    def forward(self, ctx, entry, hidden, normed=None, then=None):
        """``normed``: the first norm's rows, where the block before has left them; ``then`` = (norm, rows): the norm the next block
        starts with, to be left in ``rows``. Returns whether that was done."""
        buf = ctx.scratch("normed", tuple(hidden.shape), self.rt.dtype)
        apart = ctx.scratch("sub_out", tuple(hidden.shape), torch.float32)
        if normed is None:
            self.norms[0].forward(buf, hidden)
            normed = buf
        self.mixer.forward(ctx, (entry, 0), normed, hidden, out=apart)
        if self.feed_forward is None:
            return self._join_then(hidden, apart, self.norms[1], then)
        if not self._join_then(hidden, apart, self.norms[1], (self.norms[2], buf)):
            self.norms[2].forward(buf, hidden)
        self.feed_forward.forward(ctx, buf, hidden, out=apart)
        return self._join_then(hidden, apart, self.norms[3], then)


FUSE_SUMS = os.environ.get("ALOFA_FUSE_SUMS", "1") != "0"      # 0 (for measurements): a scaled sum into the stream and the norm behind it are two launches

register_part("block", "prenorm", PreNormBlock)
register_part("block", "scaled_prenorm", ScaledPreNormBlock)
register_part("block", "filtered_prenorm", FilteredPreNormBlock)
register_part("block", "sandwich", SandwichBlock)
