"""Block arrangements.

Pre-norm residual block: h += mixer(norm(h)); h += feed_forward(norm(h))
(src/models/qwen2/graph.rs:59-177 of yusiwen/minfer).  When only some rows are wanted after
this block (the last one of a step), they are gathered between the two halves, so the
feed-forward runs on those rows only, as the reference does for its tail rows
(graph.rs:126-138)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Block, announce_norm, normed_input, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """norms: "mixer" before the mixer, "feed_forward" before the feed-forward.  A block without a
    mixer or without a feed-forward (and then without that branch's norm) is that branch left out."""

    needs_mixer = False
    needs_feed_forward = False
    norm_names = ()
    optional_norms = ("mixer", "feed_forward")

    def __init__(self, mixer, feed_forward, norms, rt):
        super().__init__(mixer, feed_forward, norms, rt)
        for part, name in ((mixer, "mixer"), (feed_forward, "feed_forward")):
            if (part is None) != (name not in self.norms):
                raise ValueError(f"prenorm block: the {name} and the norm before it come together or not at all")

    def first_norm(self):
        return self.mixer_norm if self.mixer is not None else self.feed_forward_norm

    def forward(self, h, ctx, entry: int, writes_cache: bool, keep_rows=None):
        after = getattr(ctx, "norm_after_block", None)      # the norm that reads the stream behind this block
        if self.mixer is not None:
            x = normed_input(self.mixer_norm, self.mixer, h, ctx=ctx)
            # the mixer's output meets the feed-forward's norm, unless rows are dropped in between
            announce_norm(ctx, (self.feed_forward_norm if self.feed_forward is not None else after)
                          if keep_rows is None else None)
            self.mixer.forward(x, h, ctx, entry, writes_cache)
            ctx.norm_next = None
        if keep_rows is not None:
            kept = torch.empty((keep_rows.numel(), h.shape[1]), dtype=h.dtype, device=h.device)
            ops.gather_rows(h, keep_rows, kept)
            h = kept
        if self.feed_forward is not None:
            x = normed_input(self.feed_forward_norm, self.feed_forward, h, ctx=ctx)
            announce_norm(ctx, after)
            self.feed_forward.forward(x, h, ctx)
            ctx.norm_next = None
        return h


@register_block("branch_norm")
class BranchNormBlock(Block):
    """h += N1(mixer(h)); h += N2(feed_forward(h)): the branches read the residual stream itself
    (rounded to the run type) and only their results are normed, on the way into the stream.
    norms: "mixer_out" behind the mixer, "feed_forward_out" behind the feed-forward; a block without
    one branch has neither that branch nor its norm.

    In bfloat16 the kernel that adds a normed result into the stream also leaves the new stream
    rounded, which is the next branch's input (`ctx.stream_copy`), so no conversion runs between
    the branches of a step."""

    needs_mixer = False
    needs_feed_forward = False
    norm_names = ()
    optional_norms = ("mixer_out", "feed_forward_out")

    def __init__(self, mixer, feed_forward, norms, rt):
        super().__init__(mixer, feed_forward, norms, rt)
        for part, name in ((mixer, "mixer_out"), (feed_forward, "feed_forward_out")):
            if (part is None) != (name not in self.norms):
                raise ValueError(f"branch_norm block: a branch and the norm {name!r} behind it come together or not at all")

    def _input(self, h, ctx):
        """The stream in the run type: itself in 32-bit, else the rounded copy the last addition
        left, or a conversion."""
        if self.rt.dtype == torch.float32:
            return h
        kept = getattr(ctx, "stream_copy", None)
        if kept is not None and kept[0] is h:
            return kept[1]
        x = torch.empty(h.shape, dtype=self.rt.dtype, device=h.device)
        ops.convert(h, x)
        return x

    def _join(self, norm, y, h, ctx, want_copy: bool):
        copy = None
        if want_copy and self.rt.dtype == torch.bfloat16:
            copy = torch.empty(h.shape, dtype=torch.bfloat16, device=h.device)
        norm.add_normed(y, h, cast_out=copy)
        ctx.stream_copy = None if copy is None else (h, copy)

    @staticmethod
    def _run(part, x, rows, width, *args):
        """The branch's result as rows of their own (float32)."""
        if getattr(part, "can_overwrite", False):
            y = torch.empty((rows, width), dtype=torch.float32, device=x.device)
            part.forward(x, y, *args, accumulate=False)
        else:
            y = torch.zeros((rows, width), dtype=torch.float32, device=x.device)
            part.forward(x, y, *args)
        return y

    def forward(self, h, ctx, entry: int, writes_cache: bool, keep_rows=None):
        ctx.norm_next = ctx.norm_ahead = None
        if self.mixer is not None:
            y = self._run(self.mixer, self._input(h, ctx), h.shape[0], h.shape[1], ctx, entry, writes_cache)
            self._join(self.norms["mixer_out"], y, h, ctx, want_copy=keep_rows is None)
        if keep_rows is not None:
            kept = torch.empty((keep_rows.numel(), h.shape[1]), dtype=h.dtype, device=h.device)
            ops.gather_rows(h, keep_rows, kept)
            h = kept
        if self.feed_forward is not None:
            y = self._run(self.feed_forward, self._input(h, ctx), h.shape[0], h.shape[1], ctx)
            self._join(self.norms["feed_forward_out"], y, h, ctx, want_copy=keep_rows is None)
        return h


@register_block("sandwich")
class SandwichBlock(BranchNormBlock):
    """h += N1b(mixer(N1(h))); h += N2b(feed_forward(N2(h))): a norm before every branch and one behind it, on
    the way into the stream.  norms: "mixer" and "mixer_out" around the mixer, "feed_forward" and
    "feed_forward_out" around the feed-forward; a block without one branch has neither that branch nor its two
    norms.  The norm before a branch may stay lazy (folded into the branch's first product); the one behind it
    adds into the stream in the same kernel."""

    optional_norms = ("mixer", "mixer_out", "feed_forward", "feed_forward_out")

    def __init__(self, mixer, feed_forward, norms, rt):
        Block.__init__(self, mixer, feed_forward, norms, rt)
        for part, names in ((mixer, ("mixer", "mixer_out")), (feed_forward, ("feed_forward", "feed_forward_out"))):
            for name in names:
                if (part is None) != (name not in self.norms):
                    raise ValueError(f"sandwich block: a branch and the norms around it come together or not at all "
                                     f"({name!r})")

    def forward(self, h, ctx, entry: int, writes_cache: bool, keep_rows=None):
        ctx.norm_next = ctx.norm_ahead = None
        if self.mixer is not None:
            x = normed_input(self.norms["mixer"], self.mixer, h)
            y = self._run(self.mixer, x, h.shape[0], h.shape[1], ctx, entry, writes_cache)
            self.norms["mixer_out"].add_normed(y, h)
        if keep_rows is not None:
            kept = torch.empty((keep_rows.numel(), h.shape[1]), dtype=h.dtype, device=h.device)
            ops.gather_rows(h, keep_rows, kept)
            h = kept
        if self.feed_forward is not None:
            x = normed_input(self.norms["feed_forward"], self.feed_forward, h)
            y = self._run(self.feed_forward, x, h.shape[0], h.shape[1], ctx)
            self.norms["feed_forward_out"].add_normed(y, h)
        return h


@register_block("parallel_shared_norm")
class SharedNormParallelBlock(Block):
    """x + mixer(N(x)) + feed_forward(N(x)): one norm, whose output both branches read.  norms: "input"; a block
    without a feed-forward is the mixer's branch alone.  The normed rows are made once, before the mixer adds
    into the stream; where only some rows go on behind this block, the feed-forward gets the norm of those."""

    needs_mixer = True
    needs_feed_forward = False
    norm_names = ("input",)

    def first_norm(self):
        return self.norms["input"]

    def forward(self, h, ctx, entry: int, writes_cache: bool, keep_rows=None):
        ctx.norm_next = ctx.norm_ahead = None
        norm = self.norms["input"]
        x = norm.forward(h)
        x_ff = None
        if self.feed_forward is not None:
            x_ff = x if keep_rows is None else norm.forward(h, row_idx=keep_rows)
        self.mixer.forward(x, h, ctx, entry, writes_cache)
        if keep_rows is not None:
            kept = torch.empty((keep_rows.numel(), h.shape[1]), dtype=h.dtype, device=h.device)
            ops.gather_rows(h, keep_rows, kept)
            h = kept
        if self.feed_forward is not None:
            self.feed_forward.forward(x_ff, h, ctx)
        return h


@register_block("parallel")
class ParallelBlock(Block):
    """x + mixer(N1(x)) + feed_forward(N2(x)): both branches read the same x, each through a norm of
    its own.  norms: "mixer" before the mixer, "feed_forward" before the feed-forward; a block without
    a feed-forward has neither it nor its norm.  With a combiner, what goes on is what the combiner
    makes of the block's result (`Combiner.enter` / `leave`).

    The feed-forward's input is normed before the mixer adds into the stream; the mixer's own input
    may stay lazy (its first product reads the stream before its last one writes)."""

    needs_mixer = True
    needs_feed_forward = False
    norm_names = ("mixer",)
    optional_norms = ("feed_forward",)
    takes_combiner = True

    def __init__(self, mixer, feed_forward, norms, rt, combiner=None):
        super().__init__(mixer, feed_forward, norms, rt, combiner=combiner)
        if (feed_forward is None) != ("feed_forward" not in self.norms):
            raise ValueError("parallel block: the feed-forward and the norm before it come together or not at all")

    def forward(self, h, ctx, entry: int, writes_cache: bool, keep_rows=None):
        ctx.norm_next = ctx.norm_ahead = None
        if self.combiner is not None:
            h = self.combiner.enter(h, ctx)
        x_ff = None
        if self.feed_forward is not None:
            x_ff = self.norms["feed_forward"].forward(h, row_idx=keep_rows)
        x = normed_input(self.norms["mixer"], self.mixer, h)
        self.mixer.forward(x, h, ctx, entry, writes_cache)
        if keep_rows is not None:
            kept = torch.empty((keep_rows.numel(), h.shape[1]), dtype=h.dtype, device=h.device)
            ops.gather_rows(h, keep_rows, kept)
            h = kept
        if self.feed_forward is not None:
            self.feed_forward.forward(x_ff, h, ctx)
        if self.combiner is not None:
            h = self.combiner.leave(h, ctx, keep_rows)
        return h
