"""A second input from the tokens themselves, added to the residual stream after a layer's sublayers (category
``token_input``).

``gated_table``: a second table holds ``columns`` values per token; a layer reads ``dim`` of them from column
``column`` on, t, and adds

    y = P (gelu_tanh(G x) * t),     h <- h + y / sqrt(mean(y^2) + eps) * w

with x the stream as it stands (rounded once to the compute dtype for the product), G [dim, width], P [width, dim]
and w [width].  The table belongs to the embedding (its ``extra_tables``); this part names it as the fallback of its
own tensor, so that all layers and the embedding share one buffer.  The norm and the add into the stream are fp32
(``RMSNorm.add_normed``).
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import torch

from ..kernels import api as K
from .base import Part, Runtime, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights
from .rmsnorm import RMSNorm


class GatedTableInput(Part):
    category = "token_input"
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, vocab_size: int, dim: int, column: int, columns: int, eps: float,
                 table: str, names: Sequence[str] = ("table", "gate", "proj", "norm"), init_std: float = 0.02):
        """``table``: the full name of the table's tensor; ``names``: the local names of this part's view of the table,
        of G, P and w."""
        super().__init__(rt)
        self.hidden_size, self.vocab_size, self.dim = int(hidden_size), int(vocab_size), int(dim)
        self.column, self.columns, self.table_name = int(column), int(columns), str(table)
        if not 0 <= self.column <= self.columns - self.dim:
            raise ValueError(f"token input: columns {self.column} .. {self.column + self.dim} lie outside the table's {self.columns}")
        self.names, self.init_std = tuple(names), init_std
        self.norm = RMSNorm(rt, self.hidden_size, eps, init=("uniform", 0.5, 1.5), name=self.names[3])
        self.table: Optional[torch.Tensor] = None
        self.w_gate: Optional[torch.Tensor] = None
        self.w_proj: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        t, g, p, _ = self.names
        out = {t: WeightSpec((self.vocab_size, self.columns), fallback=self.table_name, write_when_random=False),
               g: WeightSpec((self.dim, self.hidden_size), ("normal", self.init_std)),
               p: WeightSpec((self.hidden_size, self.dim), ("normal", self.dim ** -0.5))}
        out.update(self.norm.weights())
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        t, g, p, n = self.names
        self.table = tensors[t]
        if not self.table.is_contiguous():
            self.table = self.table.contiguous()
        self.w_gate, self.w_proj = tensors[g].contiguous(), tensors[p].contiguous()
        self.norm.load({n: tensors[n]})
        prepare_weights(self.rt, [(self.w_gate, None, False), (self.w_proj, None, True)])

    def forward(self, h: torch.Tensor, ctx: StepContext, x: Optional[torch.Tensor] = None) -> None:
        """h [N, H] fp32, added to in place.  ``x``: h rounded to the compute dtype, when the caller has it already."""
        if x is None:
            x = K.cast(h, self.rt.dtype)
        u = linear(x, self.w_gate, kernels=self.rt.kernels)
        g = K.gelu_mul_rows(u, self.table, self.column, ctx.token_ids)
        self.norm.add_normed(h, linear(g, self.w_proj, keep_split=True, kernels=self.rt.kernels))

    def stream_buffer(self, program):
        """Where the program keeps the rounded stream that this part reads."""
        return program.buffer("token_input.x", program.T * self.hidden_size * program.act_bytes)

    def native(self, program, view=None, x_ready: bool = False) -> None:
        """``program.h`` is complete (nothing pending); leaves it added to.  ``x_ready``: the rounded stream is in
        :meth:`stream_buffer` already."""
        if type(self).forward is not GatedTableInput.forward:
            H = self.hidden_size
            program.python(lambda ctx: self.forward(program.h.view(torch.float32, ctx.num_tokens, H), ctx), type(self).__name__)
            return
        from ..engine.program import STREAM
        if program.pending is not None:
            raise K.KernelError("token input: the stream must be complete before it is read")
        rt, N, T, H = self.rt, program.N, program.T, self.hidden_size
        program.keep(self.table)
        x = self.stream_buffer(program)
        if not x_ready:
            program.op("core", "ia_cast", [program.h, K.DTYPE_CODE[torch.float32], x, program.act_code, N * H, STREAM])
        u = emit_linear(program, x, N, self.w_gate, rt.dtype, None, False, "token_input.u", "token_input.gate").tensor()
        program.op("core", "ia_gelu_mul_rows", [u, u, program.act_code, self.table, K.DTYPE_CODE[self.table.dtype],
                                                self.columns, self.column, program.token_ids, self.vocab_size, N,
                                                self.dim, STREAM])
        program.pending = emit_linear(program, u, N, self.w_proj, rt.dtype, None, True, "token_input.y", "token_input.proj")
        self.norm.native_branch(program, x_out=False)


register_part("token_input", "gated_table", GatedTableInput)
