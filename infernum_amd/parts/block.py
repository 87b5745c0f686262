"""Arrangements of a layer's parts around the fp32 residual stream.

``prenorm``: h' = h + mixer(norm1(h)); h'' = h' + feed_forward(norm2(h'))
(infernum-llama/src/graph_builder.rs:453-507); without a feed-forward the layer ends after its first sublayer.  Each add is carried as a pending
delta into the next norm, which adds and normalises in one pass over the row
(the reference's add_rmsnorm fusion, infernum/src/graph/optimizer.rs:105-174,
there limited to adds with one consumer).

``branchnorm``: h' = h + norm1(mixer(h)); h'' = h' + norm2(feed_forward(h')).  The
sublayers read the residual stream itself (rounded once to the compute dtype for
their matrix products) and the norm sits on each branch's output; the
feed-forward (with its norm) may be absent.  One kernel normalises the branch,
adds it into the fp32 stream and leaves the rounded stream for the next
sublayer (``RMSNorm.add_normed``).

``sandwich``: a norm before and after each sublayer, and optionally a gate on the sublayer's result that reads what
the sublayer read:  a = norm1(h); h' = h + norm1b(gate1(a) * mixer(a));  f = norm2(h'); h'' = h' + norm2b(gate2(f) *
feed_forward(f)).  The norms after the sublayers and the gates are extra parts (``mixer_post_norm``,
``feed_forward_post_norm``: norms; ``mixer_gate``, ``feed_forward_gate``: category ``branch_gate``).  One kernel gates
the branch, normalises it, adds it into the fp32 stream and, after the mixer, leaves the feed-forward's normalised
input as well (``kernels.api.gated_norm_add``).

``parallel``: h' = h + mixer(norm1(h)) + feed_forward(norm2(h)), both norms of the same stream; optionally a part
that rewrites the stream at a later pass's entry and one that adds a token's own input after the sublayers.
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import Block, CacheView, StepContext, register_part


class PreNormBlock(Block):
    """The feed-forward (with its norm) may be absent: the layer is then its first sublayer alone.  An extra part
    ``stream_in`` (category "stream_in") rewrites the residual stream before the layer's first norm."""
    graph_safe = True

    def forward(self, h: torch.Tensor, pending: Optional[torch.Tensor], ctx: StepContext,
                cache: CacheView) -> torch.Tensor:
        stream_in = self.extra.get("stream_in")
        if stream_in is not None:
            stream_in.forward(h, pending, ctx)
            pending = None
        n = self.mixer_norm.forward(h, pending)
        a = self.mixer.forward(n, ctx, cache)
        if self.feed_forward is None:
            return a
        n = self.feed_forward_norm.forward(h, a)
        return self.feed_forward.forward(n, ctx)

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not PreNormBlock.forward:
            return super().native(program, view)
        if self.extra.get("stream_in") is not None:
            self.extra["stream_in"].native(program, None)
        self.mixer_norm.native(program, None)
        self.mixer.native(program, view)
        if self.feed_forward is not None:
            self.feed_forward_norm.native(program, None)
            self.feed_forward.native(program, None)


class BranchNormBlock(Block):
    graph_safe = True

    def _stream_rows(self, h: torch.Tensor, pending, ctx: StepContext) -> torch.Tensor:
        """The residual stream in the compute dtype: what the layer before left, or a cast of h."""
        from ..kernels import api as K
        if pending is not None:                         # a layer of another arrangement left its delta unadded
            K.residual_add(h, pending.joined(self.rt.dtype) if isinstance(pending, K.SplitSum) else pending)
            ctx.extras.pop("branchnorm.x", None)
        kept = ctx.extras.get("branchnorm.x")
        if kept is not None and kept[0] is h:
            return kept[1]
        return K.cast(h, self.rt.dtype)

    def forward(self, h: torch.Tensor, pending, ctx: StepContext, cache: CacheView):
        x = self._stream_rows(h, pending, ctx)
        a = self.mixer.forward(x, ctx, cache)
        x = torch.empty_like(x)
        self.mixer_norm.add_normed(h, a, x)
        if self.feed_forward is not None:
            f = self.feed_forward.forward(x, ctx)
            x = torch.empty_like(x)
            self.feed_forward_norm.add_normed(h, f, x)
        ctx.extras["branchnorm.x"] = (h, x)             # the next layer of this arrangement reads it
        return None

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not BranchNormBlock.forward:
            return super().native(program, view)
        from ..engine.program import STREAM
        from ..kernels import api as K
        H = program.hidden_size
        if program.pending is not None or getattr(program, "x_holds_stream", None) is not program.h:
            if program.pending is not None:
                raise K.KernelError("branchnorm after an arrangement that leaves its delta unadded is not written "
                                    "as launches")
            program.op("core", "ia_cast", [program.h, K.DTYPE_CODE[torch.float32], program.x, program.act_code,
                                           program.N * H, STREAM])
        self.mixer.native(program, view)
        self.mixer_norm.native_branch(program)
        if self.feed_forward is not None:
            self.feed_forward.native(program, None)
            self.feed_forward_norm.native_branch(program)
        program.x_holds_stream = program.h              # program.x is the stream, rounded, until a norm writes it


class SandwichBlock(Block):
    graph_safe = True

    def __init__(self, rt, mixer, feed_forward, mixer_norm, feed_forward_norm, extra):
        super().__init__(rt, mixer, feed_forward, mixer_norm, feed_forward_norm, extra)
        from .rmsnorm import RMSNorm
        for name in ("mixer_post_norm",) + (("feed_forward_post_norm",) if feed_forward is not None else ()):
            if not isinstance(self.extra.get(name), RMSNorm):
                raise ValueError(f"the sandwich arrangement needs an rmsnorm as {name!r}")
        # the feed-forward's own norm rides on the kernel that adds the mixer's branch when it is the stock norm
        self._fuse_next = (feed_forward is not None and type(feed_forward_norm) is RMSNorm
                           and feed_forward_norm.eps == self.extra["mixer_post_norm"].eps)

    def _branch(self, h, y, a, gate, post, next_norm=None):
        from ..kernels import api as K
        logits = gate.logits(a) if gate is not None else None
        x = torch.empty_like(a) if next_norm is not None else None
        K.gated_norm_add(h, y, logits, gate.bias if gate is not None else None, post.weight, post.eps,
                         next_norm.weight if next_norm is not None else None, x)
        return x

    def forward(self, h: torch.Tensor, pending, ctx: StepContext, cache: CacheView):
        a = self.mixer_norm.forward(h, pending)
        y = self.mixer.forward(a, ctx, cache)
        nxt = self.feed_forward_norm if self._fuse_next else None
        f = self._branch(h, y, a, self.extra.get("mixer_gate"), self.extra["mixer_post_norm"], nxt)
        if self.feed_forward is not None:
            if f is None:
                f = self.feed_forward_norm.forward(h, None)
            y = self.feed_forward.forward(f, ctx)
            self._branch(h, y, f, self.extra.get("feed_forward_gate"), self.extra["feed_forward_post_norm"])
        return None

    def _emit_branch(self, program, gate, post, key: str, next_norm=None) -> None:
        """``program.x`` holds what the sublayer read, ``program.pending`` its result."""
        from ..engine.program import STREAM
        from ..kernels import api as K
        H = program.hidden_size
        logits = gate.emit_logits(program, key) if gate is not None else None
        f32 = K.DTYPE_CODE[torch.float32]
        program.keep(post.weight, next_norm.weight if next_norm is not None else None,
                     gate.bias if gate is not None else None)
        galts = logits.alts if logits is not None else [None]
        for alt in program.pending.alts:
            if not alt.splits and alt.dtype != self.rt.dtype:
                raise K.KernelError("gated_norm_add: the delta must have the activations' dtype")
            code = f32 if alt.splits else program.act_code
            for galt in galts:                      # the gate's logits whole or as the parts of a split product
                if galt is not None and galt.dtype != torch.float32:
                    raise K.KernelError("gated_norm_add: the gate's logits must be fp32")
                program.op("core", "ia_gated_norm_add",
                           [program.h, alt.where, code, alt.splits or 1, program.N,
                            galt.where if galt is not None else None, f32, H, (galt.splits or 1) if galt is not None else 1,
                            program.N, gate.bias if gate is not None else None, post.weight,
                            K.DTYPE_CODE[post.weight.dtype], next_norm.weight if next_norm is not None else None,
                            K.DTYPE_CODE[next_norm.weight.dtype] if next_norm is not None else 0,
                            program.x if next_norm is not None else None, program.act_code, program.N, H,
                            float(post.eps), STREAM], alt.when & galt.when if galt is not None else alt.when)
        program.pending = None

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not SandwichBlock.forward:
            return super().native(program, view)
        self.mixer_norm.native(program, None)
        self.mixer.native(program, view)
        nxt = self.feed_forward_norm if self._fuse_next else None
        self._emit_branch(program, self.extra.get("mixer_gate"), self.extra["mixer_post_norm"], "sandwich.gate1", nxt)
        if self.feed_forward is not None:
            if nxt is None:
                self.feed_forward_norm.native(program, None)
            self.feed_forward.native(program, None)
            self._emit_branch(program, self.extra.get("feed_forward_gate"), self.extra["feed_forward_post_norm"],
                              "sandwich.gate2")


class ParallelBlock(Block):
    """Mixer and feed-forward side by side, each behind a norm of its own of the SAME stream:
    h' = h + mixer(norm1(h)) + feed_forward(norm2(h)); the feed-forward (with its norm) may be absent.  The two
    results are added into the fp32 stream one after the other.  Extra parts: ``stream_in`` (category "stream_in")
    rewrites the stream before the layer's norms, in every run of the layer but those of a repeated stretch's first
    pass; ``token_input`` (category "token_input") adds to the finished stream after the sublayers."""
    graph_safe = True

    def forward(self, h: torch.Tensor, pending, ctx: StepContext, cache: CacheView):
        from ..kernels import api as K
        stream_in = self.extra.get("stream_in")
        if stream_in is not None and cache.pass_index > 0:
            stream_in.forward(h, pending, ctx)
            pending = None
        a = self.mixer.forward(self.mixer_norm.forward(h, pending), ctx, cache)
        f = None
        if self.feed_forward is not None:
            f = self.feed_forward.forward(self.feed_forward_norm.forward(h, None), ctx)
        # both results enter the fp32 stream in one pass, which leaves the rounded stream for the token input
        side = self.extra.get("token_input")
        x = torch.empty(h.shape, dtype=self.rt.dtype, device=h.device) if side is not None else None
        K.stream_add2(h, a, f, x)
        if side is not None:
            side.forward(h, ctx, x=x)
        return None

    @staticmethod
    def _emit_add(program, a, b, x) -> None:
        """One launch per pair of forms the two results can have (a tensor, the partial sums of a split product)."""
        from ..engine.program import STREAM
        from ..kernels import api as K
        f32 = K.DTYPE_CODE[torch.float32]
        code = lambda alt: f32 if alt.splits else K.DTYPE_CODE[alt.dtype]       # noqa: E731
        for aa in a.alts:
            for bb in (b.alts if b is not None else [None]):
                program.op("core", "ia_stream_add2",
                           [program.h, aa.where, code(aa), aa.splits or 1, bb.where if bb is not None else None,
                            code(bb) if bb is not None else 0, (bb.splits or 1) if bb is not None else 1, x,
                            program.act_code if x is not None else 0, program.N, program.hidden_size, STREAM],
                           aa.when & bb.when if bb is not None else aa.when)

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not ParallelBlock.forward:
            return super().native(program, view)
        if self.extra.get("stream_in") is not None and view.pass_index > 0:
            self.extra["stream_in"].native(program, None)
        self.mixer_norm.native(program, None)
        self.mixer.native(program, view)
        a, program.pending = program.pending, None
        f = None
        if self.feed_forward is not None:
            self.feed_forward_norm.native(program, None)          # nothing pending: the norm of the same stream
            self.feed_forward.native(program, None)
            f, program.pending = program.pending, None
        side = self.extra.get("token_input")
        x = side.stream_buffer(program) if side is not None else None
        self._emit_add(program, a, f, x)
        if side is not None:
            side.native(program, None, x_ready=True)


register_part("block", "prenorm", PreNormBlock)
register_part("block", "parallel", ParallelBlock)
register_part("block", "branchnorm", BranchNormBlock)
register_part("block", "sandwich", SandwichBlock)
