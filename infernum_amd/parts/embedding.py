"""Token embedding and output head.

h[t] = E[ids[t]] (infernum-llama/src/graph_builder.rs:442; times ``scale`` where a model has one);
logits = f W^T for the wanted rows only, in fp32 straight from the fp32
accumulators (:533-536).  When the file has no head matrix, the embedding
matrix stands in: the reference decides that by the file's contents, not by
``tie_word_embeddings`` (infernum-cuda/src/inner/cuda_graph_engine.rs:225-232);
the two then share one buffer here.
"""
from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import api as K
from .base import Embedding, Head, Runtime, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear


EMBEDDING_OUTPUT = "embedding.out"
EMBEDDING_OUTPUT_F32 = "embedding.out.f32"      # with keep_output="fp32": the rows as they entered the stream, unrounded


class TokenEmbedding(Embedding):
    graph_safe = True
    def __init__(self, rt: Runtime, vocab_size: int, hidden_size: int, init_std: float = 0.02, scale: float = 1.0,
                 name: str = "weight", keep_output: Any = False, position_table: Optional[Mapping[str, Any]] = None,
                 extra_tables: Optional[Mapping[str, Any]] = None):
        """``position_table`` {name, rows, init_std}: a learned vector per position, added (unscaled) to the token's row;
        a position beyond its rows leaves NaN.  ``scale`` multiplies the looked-up row in fp32 (the table itself stays as stored: a head tied to it
        reads it unscaled); ``name`` is the table's local tensor name.  ``keep_output``: the rows as they leave
        here stay available to later parts of the step, rounded to the compute dtype (``EMBEDDING_OUTPUT`` in
        ``ctx.extras``, or the program's buffer of that name); ``keep_output="fp32"`` keeps them unrounded
        (``EMBEDDING_OUTPUT_F32``).  ``extra_tables`` {local name: {cols, init_std}}: further tables with a row per
        token that this part owns and other parts read (they name the tensor as their fallback)."""
        super().__init__(rt)
        self.keep_f32 = keep_output == "fp32"
        self.keep_output = bool(keep_output) and not self.keep_f32
        self.extra_tables = {k: dict(v) for k, v in (extra_tables or {}).items()}
        self.tables: Dict[str, torch.Tensor] = {}
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.init_std = init_std
        self.scale, self.name = float(scale), str(name)
        self.table: Optional[torch.Tensor] = None
        self.position_table = dict(position_table) if position_table else None
        self.pos_rows: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        out = {self.name: WeightSpec((self.vocab_size, self.hidden_size), ("normal", self.init_std))}
        if self.position_table:
            out[self.position_table["name"]] = WeightSpec((int(self.position_table["rows"]), self.hidden_size),
                                                          ("normal", self.position_table.get("init_std", self.init_std)))
        for name, t in self.extra_tables.items():
            out[name] = WeightSpec((self.vocab_size, int(t["cols"])), ("normal", t.get("init_std", self.init_std)))
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.name].contiguous()
        if self.position_table:
            self.pos_rows = tensors[self.position_table["name"]].contiguous()
        self.tables = {name: tensors[name] for name in self.extra_tables}

    def forward(self, ctx: StepContext) -> torch.Tensor:
        h = torch.empty((ctx.num_tokens, self.hidden_size), dtype=torch.float32, device=self.table.device)
        K.embed(self.table, ctx.token_ids, h, self.scale)
        if self.pos_rows is not None:
            K.add_rows(h, self.pos_rows, ctx.positions)
        if self.keep_output:
            ctx.extras[EMBEDDING_OUTPUT] = K.cast(h, self.rt.dtype)
        if self.keep_f32:
            ctx.extras[EMBEDDING_OUTPUT_F32] = K.cast(h, torch.float32, out=torch.empty_like(h))
        return h

    def native(self, program, view=None) -> None:
        if type(self).forward is not TokenEmbedding.forward:
            return super().native(program, view)
        from ..engine.program import STREAM
        program.op("core", "ia_embed", [self.table, K.DTYPE_CODE[self.table.dtype], program.token_ids, program.h,
                                        program.N, self.hidden_size, self.vocab_size, float(self.scale), STREAM])
        if self.pos_rows is not None:
            program.op("core", "ia_add_rows", [program.h, self.pos_rows, K.DTYPE_CODE[self.pos_rows.dtype],
                                               program.positions, program.N, self.hidden_size,
                                               int(self.pos_rows.shape[0]), STREAM])
        if self.keep_output:
            kept = program.buffer(EMBEDDING_OUTPUT, program.T * self.hidden_size * program.act_bytes)
            program.op("core", "ia_cast", [program.h, K.DTYPE_CODE[torch.float32], kept, program.act_code,
                                           program.N * self.hidden_size, STREAM])
        if self.keep_f32:
            kept = program.buffer(EMBEDDING_OUTPUT_F32, program.T * self.hidden_size * 4)
            f32 = K.DTYPE_CODE[torch.float32]
            program.op("core", "ia_cast", [program.h, f32, kept, f32, program.N * self.hidden_size, STREAM])
        program.pending = None


class LinearHead(Head):
    graph_safe = True
    def __init__(self, rt: Runtime, vocab_size: int, hidden_size: int, fallback: Optional[str] = None,
                 tied: bool = False, init_std: float = 0.02, name: str = "weight", softcap: Optional[float] = None,
                 scale: float = 1.0):
        """``scale`` s: the logits are multiplied by s (in fp32).  ``softcap`` c: the logits become c tanh(logits / c).  ``name``: the matrix's local tensor name."""
        super().__init__(rt)
        self.name = str(name)
        self.softcap = float(softcap) if softcap else 0.0
        self.scale = float(scale)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.fallback, self.tied, self.init_std = fallback, bool(tied), init_std
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        return {self.name: WeightSpec((self.vocab_size, self.hidden_size), ("normal", self.init_std),
                                     fallback=self.fallback, write_when_random=not self.tied)}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        # no second copy laid out for the weight-streaming kernel: since that kernel's tiles of rows walk K from
        # starts of their own, the file's layout serves the head as well (128,256 x 4,096 on an MI355X: 187.1 against
        # 187.6 us at 8 rows, 190.0 against 189.0 at 16), and a copy would be another gigabyte
        self.weight = tensors[self.name]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = linear(x, self.weight, out_dtype=torch.float32, kernels=self.rt.kernels)
        if self.scale != 1.0 and logits.shape[0]:
            logits = K.scale_(logits if logits.is_contiguous() else logits.contiguous(), self.scale)
        if self.softcap and logits.shape[0]:
            logits = K.softcap(logits if logits.is_contiguous() else logits.contiguous(), self.softcap)
        return logits

    def native(self, program, view=None) -> None:
        if type(self).forward is not LinearHead.forward:
            return super().native(program, view)
        emit_linear(program, program.x, program.R, self.weight, torch.float32, None, False, program.logits, "head")
        from ..engine.program import STREAM
        if self.scale != 1.0:
            program.op("core", "ia_scale", [program.logits, program.R, self.vocab_size, float(self.scale), STREAM])
        if self.softcap:
            program.op("core", "ia_softcap", [program.logits, program.R, self.vocab_size, float(self.softcap), STREAM])


register_part("embedding", "token", TokenEmbedding)
register_part("head", "linear", LinearHead)
