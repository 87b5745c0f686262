"""Parts that rewrite the residual stream where a run of layers begins (category ``stream_in``).

``concat_linear``: h <- L [h ; e], with e the embedding's output of the step's tokens and L a [width, 2 width] matrix
whose first width columns meet h.  A model that runs some of its layers several times in a row starts every pass so,
which lets each pass see the tokens themselves again.  What a layer before left unadded (the pending delta) is added
into h first; the product's operands are rounded to the compute dtype like any product's, its sums and the new stream
are fp32.  The embedding must have been made with ``keep_output``.

``add_embedding``: h <- h + e, nothing else.
"""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from ..kernels import api as K
from .base import Part, Runtime, StepContext, WeightSpec, register_part
from .embedding import EMBEDDING_OUTPUT, EMBEDDING_OUTPUT_F32
from .linear import emit_linear, linear, prepare_weights


class ConcatLinearStreamIn(Part):
    category = "stream_in"
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, name: str = "weight", init_std: float = 0.02):
        super().__init__(rt)
        self.hidden_size, self.name, self.init_std = int(hidden_size), str(name), init_std
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        H = self.hidden_size
        return {self.name: WeightSpec((H, 2 * H), ("normal", self.init_std))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name].contiguous()
        prepare_weights(self.rt, [(self.weight, None, False)])

    def forward(self, h: torch.Tensor, pending: Any, ctx: StepContext) -> None:
        """h [N, H] fp32, rewritten in place."""
        e = ctx.extras.get(EMBEDDING_OUTPUT)
        if e is None:
            raise K.KernelError("concat_linear: the embedding did not keep its output (keep_output)")
        if pending is not None:
            K.stream_add(h, pending)
        both = K.concat_cast(h, e)
        h.copy_(linear(both, self.weight, out_dtype=torch.float32, kernels=self.rt.kernels))

    def native(self, program, view=None) -> None:
        if type(self).forward is not ConcatLinearStreamIn.forward:
            H, pending = self.hidden_size, program.pending
            program.python(lambda ctx: self.forward(program.h.view(torch.float32, ctx.num_tokens, H),
                                                    program.read(pending, ctx.num_tokens), ctx), type(self).__name__)
            program.pending = None
            return
        from ..engine.program import STREAM
        H, T, N = self.hidden_size, program.T, program.N
        for alt in (program.pending.alts if program.pending is not None else []):
            code = K.DTYPE_CODE[torch.float32] if alt.splits else K.DTYPE_CODE[alt.dtype]
            program.op("core", "ia_stream_add", [program.h, alt.where, code, alt.splits or 1, N, H, STREAM], alt.when)
        program.pending = None
        kept = program.buffer(EMBEDDING_OUTPUT, T * H * program.act_bytes)
        both = program.buffer("stream_in.both", T * 2 * H * program.act_bytes)
        program.op("core", "ia_concat_cast", [program.h, kept, both, program.act_code, N, H, STREAM])
        emit_linear(program, both, N, self.weight, torch.float32, None, False, program.h, "stream_in")


class AddEmbeddingStreamIn(Part):
    """h <- h + e: the embedding's rows of the step's tokens, as they first entered the stream (fp32, unrounded),
    are added again.  No tensors.  The embedding must have been made with ``keep_output="fp32"``."""
    category = "stream_in"
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int):
        super().__init__(rt)
        self.hidden_size = int(hidden_size)

    def forward(self, h: torch.Tensor, pending: Any, ctx: StepContext) -> None:
        e = ctx.extras.get(EMBEDDING_OUTPUT_F32)
        if e is None:
            raise K.KernelError("add_embedding: the embedding did not keep its output (keep_output='fp32')")
        if pending is not None:
            K.stream_add(h, pending)
        K.stream_add(h, e)

    def native(self, program, view=None) -> None:
        from ..engine.program import STREAM
        H, N = self.hidden_size, program.N
        f32 = K.DTYPE_CODE[torch.float32]
        for alt in (program.pending.alts if program.pending is not None else []):
            code = f32 if alt.splits else K.DTYPE_CODE[alt.dtype]
            program.op("core", "ia_stream_add", [program.h, alt.where, code, alt.splits or 1, N, H, STREAM], alt.when)
        program.pending = None
        kept = program.buffer(EMBEDDING_OUTPUT_F32, program.T * H * 4)
        program.op("core", "ia_stream_add", [program.h, kept, f32, 1, N, H, STREAM])


register_part("stream_in", "concat_linear", ConcatLinearStreamIn)
register_part("stream_in", "add_embedding", AddEmbeddingStreamIn)
