"""Block arrangements: where the norms stand around mixers and feed-forwards.

An arrangement names its parts itself: SLOTS maps each part's name in the block to its kind ("norm",
"mixer", "feed_forward").  A layer's description gives a part for every slot; the model builds them
from the parts' registries and hands them to the arrangement's constructor by those names.  The
arrangement says which of them keep caches (`mixers()`, in the order in which a LayerCall lists their
caches) and runs them (`forward(x, ctx, caches, runtime)`, `caches` in that same order)."""
from __future__ import annotations

from ..kernels import ops
import torch

from .base import ARRANGEMENTS, DeferredSum, LazyNorm, StreamStats


@ARRANGEMENTS.register("pre_norm")
class PreNormBlock:
    """x += mixer(norm1(x)); x += ffn(norm2(x))     (crates/denno-engine/src/model/gpt2.rs:152-220)"""

    SLOTS = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ffn": "feed_forward"}

    def __init__(self, norm1, mixer, norm2, ffn):
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn

    def parts(self):
        return [self.norm1, self.mixer, self.norm2, self.ffn]

    def mixers(self):
        return [self.mixer]

    def first_norm(self):
        """The norm that reads the residual stream first in this block."""
        return self.norm1

    def after_bind(self):
        self.mixer.prepare_lazy_norm(self.norm1)
        self.ffn.prepare_lazy_norm(self.norm2)

    takes_deferred = True     # its first norm adds what the block before left in Runtime.stream_deferred

    def forward(self, x, ctx, caches, runtime):
        cache = caches[0]
        # A product into the stream may leave its sum for the kernel of the norm behind it (steps of 65 to 256
        # rows, few columns: parts.base.DeferredSum): the part before a norm is offered an empty one, the norm gets
        # what was put there; across blocks it travels in runtime.stream_deferred.
        came = runtime.stream_deferred
        runtime.stream_deferred = None
        can = runtime.deferred_sums
        mid = DeferredSum() if can and getattr(self.norm2, "adds_deferred", False) and self.mixer.defers_sum(x.shape[0]) else None
        end = (DeferredSum() if can and getattr(runtime.next_norm, "adds_deferred", False) and runtime.next_takes_deferred
               and self.ffn.defers_sum(x.shape[0]) else None)
        # A norm is a kernel of its own, or, where the parts on both sides of it can (steps of few
        # rows), it runs inside them: the part before leaves what the norm needs as it adds into the
        # stream, the part after applies it in its own kernel (parts.base.StreamStats, LazyNorm).
        n = x.shape[0] if runtime.norms_inside_products else 1 << 30      # (so many rows nobody takes)
        before = runtime.stream_stats
        if before is not None and not (before.written and before.norm is self.norm1
                                       and self.mixer.takes_lazy_norm(n, self.norm1)):
            before = None
        between = (self._stats(x, self.norm2)
                   if self.mixer.writes_norm_stats(n) and self.ffn.takes_lazy_norm(n, self.norm2) else None)
        nxt = runtime.next_norm
        after = self._stats(x, nxt) if nxt is not None and self.ffn.writes_norm_stats(n) else None
        runtime.stream_stats = None
        self.mixer.forward(self._normed(self.norm1, x, self.mixer, before, runtime, came), ctx, cache, accumulate_into=x,
                           **({"stats": between} if between is not None else {}),
                           **({"deferred": mid} if mid is not None else {}))
        if between is not None and not between.written:
            between = None
        self.ffn.forward(self._normed(self.norm2, x, self.ffn, between, runtime, mid), ctx, accumulate_into=x,
                         **({"stats": after} if after is not None else {}),
                         **({"deferred": end} if end is not None else {}))
        runtime.stream_stats = after if after is not None and after.written else None
        runtime.stream_deferred = end if end is not None and end.filled else None

    @staticmethod
    def _stats(x, norm):
        if getattr(norm, "fused_params", None) is None:
            return None
        return StreamStats(*ops.norm_stream_buffers(x.shape[0], x.shape[1], x.device), norm)

    @staticmethod
    def _normed(norm, x, part, stream, runtime, deferred=None):
        """The rows that `part` reads: normed here, or left to the part's own first kernel.  deferred: a sum that
        is not in the stream yet: the norm's kernel adds it, or it is added first."""
        if deferred is not None and deferred.filled:
            if getattr(norm, "adds_deferred", False) and stream is None:
                return norm.forward(x, runtime.act_dtype, packed=part.packed_input(x.shape[0]), deferred=deferred)
            deferred.flush(x)
        if stream is not None:
            return LazyNorm(norm, x, runtime.act_dtype, stream)
        return norm.forward(x, runtime.act_dtype, packed=part.packed_input(x.shape[0]))


@ARRANGEMENTS.register("pre_norm_filtered")
class FilteredPreNormBlock:
    """x += mixer(filter(norm1(x))); x += ffn(norm2(x)).  The filter (a short convolution over time, or none) reads the
    normed rows in 32-bit and keeps a state of its own, so a call of this block names two caches: the filter's and the
    mixer's.  A block whose feed-forward is "none" ends after the mixer."""

    SLOTS = {"norm1": "norm", "filter": "filter", "mixer": "mixer", "norm2": "norm", "ffn": "feed_forward"}

    def __init__(self, norm1, filter, mixer, norm2, ffn):
        self.norm1, self.filter, self.mixer, self.norm2, self.ffn = norm1, filter, mixer, norm2, ffn
        self.has_ffn = not getattr(ffn, "absent", False)

    def parts(self):
        return [self.norm1, self.filter, self.mixer] + ([self.norm2, self.ffn] if self.has_ffn else [])

    def mixers(self):
        return [self.filter, self.mixer]

    def forward(self, x, ctx, caches, runtime):
        runtime.stream_stats = None
        h = self.norm1.forward(x, getattr(self.filter, "in_dtype", runtime.act_dtype))
        h = self.filter.forward(h, ctx, caches[0])
        self.mixer.forward(h, ctx, caches[1], accumulate_into=x)
        if self.has_ffn:
            self.ffn.forward(self.norm2.forward(x, runtime.act_dtype), ctx, accumulate_into=x)


@ARRANGEMENTS.register("pre_norm_plain")
class PlainPreNormBlock:
    """x += mixer(norm1(x)); x += ffn(norm2(x)), every norm a kernel of its own.  The mixer may be several side by side
    (its `cache_parts`: a call of this block then names a cache for each).  A block whose feed-forward is "none" ends after
    the mixer."""

    SLOTS = {"norm1": "norm", "mixer": "mixer", "norm2": "norm", "ffn": "feed_forward"}

    def __init__(self, norm1, mixer, norm2, ffn):
        self.norm1, self.mixer, self.norm2, self.ffn = norm1, mixer, norm2, ffn
        self.has_ffn = not getattr(ffn, "absent", False)

    def parts(self):
        return [self.norm1, self.mixer] + ([self.norm2, self.ffn] if self.has_ffn else [])

    def mixers(self):
        return self.mixer.cache_parts()

    def forward(self, x, ctx, caches, runtime):
        runtime.stream_stats = None
        self.mixer.forward(self.norm1.forward(x, runtime.act_dtype), ctx, caches if len(caches) != 1 else caches[0], accumulate_into=x)
        if self.has_ffn:
            self.ffn.forward(self.norm2.forward(x, runtime.act_dtype), ctx, accumulate_into=x)


@ARRANGEMENTS.register("sandwich")
class SandwichBlock:
    """A norm before and a norm behind each sublayer: x += post1(mixer(norm1(x))); x += post2(ffn(norm2(x))).  The norms
    behind are of a kind that adds into the stream itself (`add_into(y, x)`, parts.norms.StreamRMSNorm: a multiplier of
    the model and a vector of the layer ride along).  A block whose feed-forward is "none" ends after the mixer."""

    SLOTS = {"norm1": "norm", "mixer": "mixer", "post1": "norm", "norm2": "norm", "ffn": "feed_forward", "post2": "norm"}

    def __init__(self, norm1, mixer, post1, norm2, ffn, post2):
        self.norm1, self.mixer, self.post1, self.norm2, self.ffn, self.post2 = norm1, mixer, post1, norm2, ffn, post2
        self.has_ffn = not getattr(ffn, "absent", False)
        for n in (post1, post2):
            if not hasattr(n, "add_into"):
                raise TypeError(f"sandwich: the norm behind a sublayer must add into the stream; {type(n).__name__} does not")

    def parts(self):
        return [self.norm1, self.mixer, self.post1] + ([self.norm2, self.ffn, self.post2] if self.has_ffn else [])

    def mixers(self):
        return [self.mixer]

    @staticmethod
    def _result(part, x, *args):
        """The sublayer's result as 32-bit rows of its own: from a part that can return them (`returns_rows`), or
        added by the part into rows of zeros."""
        if getattr(part, "returns_rows", False):
            return part.forward(*args, accumulate_into=None)
        y = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        part.forward(*args, accumulate_into=y)
        return y

    def forward(self, x, ctx, caches, runtime):
        runtime.stream_stats = None
        h = self.norm1.forward(x, runtime.act_dtype)
        self.post1.add_into(self._result(self.mixer, x, h, ctx, caches[0]), x)
        if self.has_ffn:
            h = self.norm2.forward(x, runtime.act_dtype)
            self.post2.add_into(self._result(self.ffn, x, h, ctx), x)


@ARRANGEMENTS.register("gated_sandwich")
class GatedSandwichBlock(SandwichBlock):
    """The sandwich with a gate on each sublayer's result and a token input at the end: with h = norm1(x),
    x += post1(mixer(h) * sigmoid(gate1(h))); with h = norm2(x), x += post2(ffn(h) * sigmoid(gate2(h))); then the token
    input adds what the rows' tokens pick (parts.token_inputs).  A gate reads the rows its sublayer read; the
    multiplication runs inside the kernel of the norm behind.  Gates and token input may be "none"; a block whose
    feed-forward is "none" goes from the mixer straight to the token input."""

    SLOTS = {"norm1": "norm", "mixer": "mixer", "gate1": "gate", "post1": "norm", "norm2": "norm", "ffn": "feed_forward",
             "gate2": "gate", "post2": "norm", "side": "token_input"}

    def __init__(self, norm1, mixer, gate1, post1, norm2, ffn, gate2, post2, side):
        super().__init__(norm1, mixer, post1, norm2, ffn, post2)
        self.gate1, self.gate2, self.side = gate1, gate2, side
        self.has_side = not getattr(side, "absent", False)

    def parts(self):
        return ([self.norm1, self.mixer, self.gate1, self.post1]
                + ([self.norm2, self.ffn, self.gate2, self.post2] if self.has_ffn else []) + ([self.side] if self.has_side else []))

    def first_norm(self):
        """The norm that reads the residual stream first in this block."""
        return self.norm1

    def forward(self, x, ctx, caches, runtime):
        # The norm in front of a sublayer is made by the kernel that takes the sublayer before into the stream (the norm
        # behind it, or the token input), where that norm is a plain one: a launch less per sublayer; across blocks the rows
        # travel in runtime.normed_rows with the norm they were made for.
        act = runtime.act_dtype
        runtime.stream_stats = None
        came, runtime.normed_rows = runtime.normed_rows, None
        h = came[1] if came is not None and came[0] is self.norm1 else self.norm1.forward(x, act)
        nxt = runtime.next_norm
        y = self._result(self.mixer, x, h, ctx, caches[0])
        then = self.norm2 if self.has_ffn else (None if self.has_side else nxt)
        h = self.post1.add_into(y, x, gate=self.gate1.logits(h), then=then, out_dtype=act)
        if self.has_ffn:
            if h is None:
                h = self.norm2.forward(x, act)
            y = self._result(self.ffn, x, h, ctx)
            h = self.post2.add_into(y, x, gate=self.gate2.logits(h), then=None if self.has_side else nxt, out_dtype=act)
        if self.has_side:
            h = self.side.forward(x, ctx, then=nxt)
        if h is not None and nxt is not None:
            runtime.normed_rows = (nxt, h)


@ARRANGEMENTS.register("multi_stream")
class MultiStreamBlock:
    """The stream is several copies (DecoderSpec.streams).  For each sublayer f (the mixer, then the feed-forward) with its
    connector c and norm: y = f(norm(c.read(copies))); c.write(copies, y) makes every copy anew.  A block whose
    feed-forward is "none" ends after the mixer.  A sublayer's result comes as 32-bit rows of its own (`returns_rows`, or
    added into rows of zeros).  The read of the sublayer that follows, in this block or the next, runs in the kernel of
    the write before it: the rows travel in `runtime.stream_rows`."""

    SLOTS = {"norm1": "norm", "hc1": "connector", "mixer": "mixer", "norm2": "norm", "hc2": "connector", "ffn": "feed_forward"}
    multi_stream = True

    def __init__(self, norm1, hc1, mixer, norm2, hc2, ffn):
        self.norm1, self.hc1, self.mixer, self.norm2, self.hc2, self.ffn = norm1, hc1, mixer, norm2, hc2, ffn
        self.has_ffn = not getattr(ffn, "absent", False)

    def parts(self):
        return [self.norm1, self.hc1, self.mixer] + ([self.norm2, self.hc2, self.ffn] if self.has_ffn else [])

    def mixers(self):
        return self.mixer.cache_parts()

    def first_read(self):
        """(connector, norm) of the sublayer that reads the stream first."""
        return self.hc1, self.norm1

    def forward(self, xs, ctx, caches, runtime):
        act = runtime.act_dtype
        runtime.stream_stats = None
        came = getattr(runtime, "stream_rows", None)      # (the block before read for this one as it wrote)
        runtime.stream_rows = None
        h = came if came is not None else self.hc1.read(xs, self.norm1, act)
        cache = caches if len(caches) != 1 else caches[0]
        # (a mixer of two branches hands both results over: their norms and their mean happen in the write's kernel)
        pair = self.mixer.forward_pair(h, ctx, caches) if hasattr(self.mixer, "forward_pair") else None
        y, branches = pair if pair is not None else (SandwichBlock._result(self.mixer, xs[0], h, ctx, cache), None)
        nxt = getattr(runtime, "next_read", None)
        if self.has_ffn:
            h = self.hc1.write(xs, y, self.hc2, self.norm2, act, branches=branches)
            y, branches = SandwichBlock._result(self.ffn, xs[0], h, ctx), None
            last = self.hc2
        else:
            last = self.hc1
        if nxt is not None:
            runtime.stream_rows = last.write(xs, y, nxt[0], nxt[1], act, branches=branches)
        else:
            last.write(xs, y, branches=branches)
