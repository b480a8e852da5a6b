"""Arrangement of a layer's parts.  `prenorm` (ampere_kv/runner.py:117-121, :165-179):
    h1 = h + mixer(norm_a(h));  h2 = h1 + feed_forward(norm_b(h1))
The residual sum `stream` is float32.  A branch's output is not added by itself: it is handed on as
`pending` and added inside the next norm's kernel, which reads the stream anyway.  In steps of few rows a branch
may instead add its output to the stream inside its last product and hand on the rows' sums of squares
(`StreamSums`); the next norm then happens inside the product that reads it, and the layer launches no norm kernel."""

from __future__ import annotations

from .base import NormedDelta, Part, ScaledDelta, Unsettled, build_part, register_part
from .base import StreamSums


class PreNormBlock(Part):
    graph_safe = True
    takes_stream_sums = True        # `pending` may be a `StreamSums`: the stream then already holds the branch's output

    def __init__(self, spec, runtime, mixer, feed_forward):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm = build_part("norm", spec["norm"], runtime)
        self.feed_forward_norm = build_part("norm", spec["norm"], runtime)
        self.mixer_norm_name = spec.get("mixer_norm_name", "input_layernorm") + ".weight"
        self.feed_forward_norm_name = spec.get("feed_forward_norm_name", "post_attention_layernorm") + ".weight"

    def tensors(self, prefix):
        return (self.mixer_norm.tensors(prefix + self.mixer_norm_name) + self.mixer.tensors(prefix)
                + self.feed_forward_norm.tensors(prefix + self.feed_forward_norm_name)
                + self.feed_forward.tensors(prefix))

    def load(self, fetch, prefix):
        self.mixer_norm.load(fetch, prefix + self.mixer_norm_name)
        self.mixer.load(fetch, prefix)
        self.feed_forward_norm.load(fetch, prefix + self.feed_forward_norm_name)
        self.feed_forward.load(fetch, prefix)

    def weight_bytes(self):
        return (self.mixer.weight_bytes() + self.feed_forward.weight_bytes()
                + self.mixer_norm.weight_bytes() + self.feed_forward_norm.weight_bytes())

    def forward(self, stream, pending, ctx, cache, writes_cache=True):
        """stream [tokens, hidden] float32 (updated in place); pending: the previous branch's output, not
        yet added, or None.  Returns this block's own pending output."""
        fold = bool(self.rt.kernels.folds_norm(stream.shape[0], self.hidden, self.rt.dtype))
        later, later_gain = ctx.fold_into_stream, ctx.fold_gain     # whoever reads this block's `pending` takes sums
        normed, unnormed = self._normed(self.mixer_norm, self.mixer, stream, pending, ctx, fold)
        ctx.fold_into_stream = fold         # the mixer's output meets this block's own second norm
        ctx.fold_gain = self.feed_forward_norm.fold_gain()
        mixed = self.mixer.forward(normed, ctx, cache, writes_cache)
        stream = self._after(unnormed, stream, ctx)
        normed, unnormed = self._normed(self.feed_forward_norm, self.feed_forward, stream, mixed, ctx, fold)
        ctx.fold_into_stream = fold and later
        ctx.fold_gain = later_gain
        out = self.feed_forward.forward(normed, ctx)
        ctx.fold_into_stream = later
        self._after(unnormed, stream, ctx)
        return out

    def entry_gain(self):
        return self.mixer_norm.fold_gain()

    def _normed(self, norm, reader, stream, delta, ctx, fold=False):
        """norm(stream + delta) for `reader`: computed now - or, in steps of few rows (the context then has a spare
        buffer for the residual sum), handed on unnormed to a reader that can take that, whose first product may
        norm the rows itself: one launch less."""
        if isinstance(delta, StreamSums):    # the stream holds the branch's output already; its sums of squares are known
            unnormed = norm.scaled(stream, delta, ctx.arena) if reader.takes_pending_norm else None
            if unnormed is not None:
                return unnormed, unnormed
            normed = ctx.arena.take((stream.shape[0], self.hidden), self.rt.dtype)
            norm.forward_residual(stream, None, normed)
            return normed, None
        # (while branches add themselves to the stream it stays in its buffer: a branch finds it through the context)
        spare = None if fold else ctx.spare_stream
        if spare is not None and reader.takes_pending_norm:
            unnormed = norm.pending(stream, delta, spare, ctx.arena)
            if unnormed is not None:
                return unnormed, unnormed
        normed = ctx.arena.take((stream.shape[0], self.hidden), self.rt.dtype)
        norm.forward_residual(stream, delta, normed)
        return normed, None

    @staticmethod
    def _after(unnormed, stream, ctx):
        """Where the residual sum is after the reader ran: in the spare buffer if its product normed the rows - the two
        buffers then change roles, and the context is told - else where it was."""
        if unnormed is None or not unnormed.moved:
            return stream
        ctx.stream, ctx.spare_stream = unnormed.stream_out, stream
        return unnormed.stream_out


def _build_prenorm(spec, runtime, mixer=None, feed_forward=None):
    return PreNormBlock(spec, runtime, mixer, feed_forward)


register_part("block", "prenorm", _build_prenorm)


class SandwichBlock(Part):
    """Every branch is normed before and after:
        h1 = h + norm_b(mixer(norm_a(h)));  h2 = h1 + norm_d(feed_forward(norm_c(h1)))
    (a layer without a feed-forward ends after the first line).  The norm after a branch, the addition to the float32
    residual sum and the norm before the next branch are one kernel (`Norm.after`); the last branch of the block is
    handed on as a `NormedDelta` and meets the next block's first norm - or the model's end - the same way."""
    graph_safe = True
    takes_normed_delta = True

    def __init__(self, spec, runtime, mixer, feed_forward):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.mixer, self.feed_forward = mixer, feed_forward
        self.has_feed_forward = not isinstance(feed_forward, NoFeedForward)
        names = tuple(spec.get("names", ("norm1", "norm1b", "norm2", "norm2b")))
        if len(names) != 4:
            raise ValueError(f"a block of four norms needs four names, got {names}")
        self.names = names if self.has_feed_forward else names[:2]
        self.norms = [build_part("norm", spec["norm"], runtime) for _ in self.names]

    def tensors(self, prefix):
        specs = []
        for norm, name in zip(self.norms, self.names):
            specs += norm.tensors(prefix + name)
        return specs + self.mixer.tensors(prefix) + self.feed_forward.tensors(prefix)

    def load(self, fetch, prefix):
        for norm, name in zip(self.norms, self.names):
            norm.load(fetch, prefix + name)
        self.mixer.load(fetch, prefix)
        self.feed_forward.load(fetch, prefix)

    def weight_bytes(self):
        return self.mixer.weight_bytes() + self.feed_forward.weight_bytes() + sum(n.weight_bytes() for n in self.norms)

    def forward(self, stream, pending, ctx, cache, writes_cache=True):
        if pending is not None and not isinstance(pending, Unsettled):
            raise TypeError("a block of four norms is handed a branch that is still to be added, or nothing")
        ctx.fold_into_stream, ctx.fold_gain = False, None      # no branch of this block adds itself to the stream
        shape = (stream.shape[0], self.hidden)
        normed = self.norms[0].after(stream, pending, ctx.arena.take(shape, self.rt.dtype))
        mixed = NormedDelta(self.mixer.forward(normed, ctx, cache, writes_cache), self.norms[1])
        if not self.has_feed_forward:
            return mixed
        normed = self.norms[2].after(stream, mixed, ctx.arena.take(shape, self.rt.dtype))
        return NormedDelta(self.feed_forward.forward(normed, ctx), self.norms[3])


class ScaledPreNormBlock(Part):
    """Pre-norm with a constant on every branch:
        h1 = h + m * mixer(norm_a(h));  h2 = h1 + m * feed_forward(norm_b(h1))
    (a layer without a feed-forward ends after the first line).  The norms are float32 up to their one rounding; the
    addition of a branch and the norm that follows are one kernel, and the block's last branch is handed on as a
    `ScaledDelta`, which the next block's first norm - or the model's end - adds the same way."""
    graph_safe = True
    takes_normed_delta = True

    def __init__(self, spec, runtime, mixer, feed_forward):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.scale = float(spec.get("residual_scale", 1.0))
        self.mixer, self.feed_forward = mixer, feed_forward
        self.has_feed_forward = not isinstance(feed_forward, NoFeedForward)
        names = tuple(spec.get("names", ("norm1", "norm2")))
        if len(names) != 2:
            raise ValueError(f"a pre-norm block has two norms, got the names {names}")
        self.names = names if self.has_feed_forward else names[:1]
        self.norms = [build_part("norm", spec["norm"], runtime) for _ in self.names]

    def tensors(self, prefix):
        specs = []
        for norm, name in zip(self.norms, self.names):
            specs += norm.tensors(prefix + name)
        return specs + self.mixer.tensors(prefix) + self.feed_forward.tensors(prefix)

    def load(self, fetch, prefix):
        for norm, name in zip(self.norms, self.names):
            norm.load(fetch, prefix + name)
        self.mixer.load(fetch, prefix)
        self.feed_forward.load(fetch, prefix)

    def weight_bytes(self):
        return self.mixer.weight_bytes() + self.feed_forward.weight_bytes() + sum(n.weight_bytes() for n in self.norms)

    def forward(self, stream, pending, ctx, cache, writes_cache=True):
        if pending is not None and not isinstance(pending, Unsettled):
            raise TypeError("a scaled pre-norm block is handed a branch that is still to be added, or nothing")
        ctx.fold_into_stream, ctx.fold_gain = False, None      # no branch of this block adds itself to the stream
        shape = (stream.shape[0], self.hidden)
        normed = self.norms[0].after(stream, pending, ctx.arena.take(shape, self.rt.dtype))
        mixed = ScaledDelta(self.mixer.forward(normed, ctx, cache, writes_cache), self.scale, self.rt.kernels)
        if not self.has_feed_forward:
            return mixed
        normed = self.norms[1].after(stream, mixed, ctx.arena.take(shape, self.rt.dtype))
        return ScaledDelta(self.feed_forward.forward(normed, ctx), self.scale, self.rt.kernels)


class SharedNormBlock(Part):
    """One norm, and both branches read its output:
        n = norm(h);  h' = h + m * (mixer(n) + feed_forward(n))
    (a layer without a feed-forward adds the mixer alone).  The norm is float32 up to its one rounding; the two outputs
    travel on together as one `ScaledDelta` and are added - to each other in float32, then to the residual sum - inside
    the kernel of the next block's norm, or at the model's end."""
    graph_safe = True
    takes_normed_delta = True

    def __init__(self, spec, runtime, mixer, feed_forward):
        self.rt = runtime
        self.hidden = int(spec["hidden_size"])
        self.scale = float(spec.get("residual_scale", 1.0))
        self.mixer, self.feed_forward = mixer, feed_forward
        self.has_feed_forward = not isinstance(feed_forward, NoFeedForward)
        self.name = spec.get("name", "norm1")
        self.norm = build_part("norm", spec["norm"], runtime)

    def tensors(self, prefix):
        return self.norm.tensors(prefix + self.name) + self.mixer.tensors(prefix) + self.feed_forward.tensors(prefix)

    def load(self, fetch, prefix):
        self.norm.load(fetch, prefix + self.name)
        self.mixer.load(fetch, prefix)
        self.feed_forward.load(fetch, prefix)

    def weight_bytes(self):
        return self.mixer.weight_bytes() + self.feed_forward.weight_bytes() + self.norm.weight_bytes()

    def forward(self, stream, pending, ctx, cache, writes_cache=True):
        if pending is not None and not isinstance(pending, Unsettled):
            raise TypeError("a block with one norm is handed a branch that is still to be added, or nothing")
        ctx.fold_into_stream, ctx.fold_gain = False, None      # no branch of this block adds itself to the stream
        normed = self.norm.after(stream, pending, ctx.arena.take((stream.shape[0], self.hidden), self.rt.dtype))
        mixed = self.mixer.forward(normed, ctx, cache, writes_cache)
        other = self.feed_forward.forward(normed, ctx) if self.has_feed_forward else None
        return ScaledDelta(mixed, self.scale, self.rt.kernels, second=other)


class NoFeedForward(Part):
    """The feed-forward of a layer that has none."""
    graph_safe = True

    def __init__(self, spec=None, runtime=None):
        pass


register_part("block", "sandwich", lambda spec, runtime, mixer=None, feed_forward=None:
              SandwichBlock(spec, runtime, mixer, feed_forward))
register_part("block", "scaled_prenorm", lambda spec, runtime, mixer=None, feed_forward=None:
              ScaledPreNormBlock(spec, runtime, mixer, feed_forward))
register_part("block", "shared_norm", lambda spec, runtime, mixer=None, feed_forward=None:
              SharedNormBlock(spec, runtime, mixer, feed_forward))
register_part("feed_forward", "none", NoFeedForward)
