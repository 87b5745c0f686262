"""RMSNorm on the fp32 residual stream, with the residual add fused in.

out = s * (1 / sqrt(mean(s^2) + eps)) * w with s = h + delta: eps inside the
root, the weight multiplies (infernum-cuda/kernels/rmsnorm.cu:79-80,89-93; fused
add: kernels/add_rmsnorm.cu:53-109).  The sum stays fp32 here, where the
reference rounds it to bf16 between the add and the norm.

Two options serve other arrangements with the same weight vector: ``unit_offset``
(the stored weight lies around zero and the norm multiplies by 1 + w), and
:meth:`RMSNorm.add_normed`, the norm on a branch's output, h += norm(delta), which
the ``branchnorm`` arrangement uses in place of ``forward``.  ``name`` is the
tensor's local name ("weight" by default; "" when the prefix is the whole name).
``scalar``: the stored weight is a single number for all values of a row.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import api as K
from .base import Norm, Runtime, WeightSpec, register_part


class RMSNorm(Norm):
    graph_safe = True
    def __init__(self, rt: Runtime, size: int, eps: float, init: tuple = ("ones",), unit_offset: bool = False,
                 name: str = "weight", scalar: bool = False):
        """``scalar``: the file holds one number, which multiplies every value of the row."""
        super().__init__(rt)
        self.scalar = bool(scalar)
        self.size = int(size)
        self.eps = float(eps)
        self.init = tuple(init)
        self.unit_offset = bool(unit_offset)
        self.name = str(name)
        self.weight: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        # a norm weight stored in fp32 stays fp32; the kernel reads either
        return {self.name: WeightSpec(() if self.scalar else (self.size,), init=self.init, follows_compute_dtype=False)}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        w = tensors[self.name].contiguous()
        if self.scalar:             # the kernels read a weight a value: the one number, as often as the row is long
            w = w.to(torch.float32).reshape(1).expand(self.size).contiguous()
        if self.unit_offset:
            w = (w.to(torch.float32) + 1.0).contiguous()       # 1 + w once, in fp32 (exact for a bf16 w)
        self.weight = w

    def add_normed(self, h: torch.Tensor, delta, x: Optional[torch.Tensor] = None) -> torch.Tensor:
        """h [N, H] fp32 += delta * rsqrt(mean(delta^2) + eps) * weight, in place; ``delta`` a tensor in the
        compute dtype or a SplitSum.  ``x`` (optional, [N, H] in the compute dtype) gets the new h."""
        return K.norm_add(h, delta, self.weight, self.eps, x)

    def native_branch(self, program, x_out: bool = True) -> None:
        """:meth:`add_normed` of ``program.pending`` into ``program.h``; the new h, rounded, goes to ``program.x``."""
        from ..engine.program import STREAM
        if program.pending is None:
            raise K.KernelError("norm on a branch: there is no branch output to normalise")
        for alt in program.pending.alts:
            if not alt.splits and alt.dtype != self.rt.dtype:
                raise K.KernelError("norm_add: the delta must have the activations' dtype")
            code = K.DTYPE_CODE[torch.float32] if alt.splits else program.act_code
            program.op("core", "ia_norm_add",
                       [program.h, alt.where, code, alt.splits or 1, program.N, self.weight,
                        K.DTYPE_CODE[self.weight.dtype], program.x if x_out else None, program.act_code, program.N,
                        self.size, float(self.eps), STREAM], alt.when)
        program.pending = None

    def forward(self, h: torch.Tensor, delta, out: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = rows.numel() if rows is not None else h.shape[0]
        if out is None:
            out = torch.empty((n, self.size), dtype=self.rt.dtype, device=h.device)
        return K.add_rmsnorm(h, delta, self.weight, self.eps, out, rows)


    def native(self, program, view=None, rows: bool = False) -> None:
        """One launch per form the pending delta can have (none, a tensor, partial sums of a split product)."""
        if type(self).forward is not RMSNorm.forward:
            return super().native(program, view, rows)          # a subclass that computes something else
        from ..engine.program import ALWAYS, STREAM, Guard
        base = Guard.between(program.R, 1) if rows else ALWAYS
        for alt in (program.pending.alts if program.pending is not None else [None]):
            delta, code, splits, when = None, program.act_code, 1, base
            if alt is not None:
                if not alt.splits and alt.dtype != self.rt.dtype:
                    raise K.KernelError("add_rmsnorm: the delta must have the activations' dtype")
                delta, when = alt.where, base & alt.when
                code, splits = (K.DTYPE_CODE[torch.float32], alt.splits) if alt.splits else (program.act_code, 1)
            program.op("core", "ia_add_rmsnorm",
                       [program.h, delta, code, splits, program.N, program.act_code, self.weight,
                        K.DTYPE_CODE[self.weight.dtype], program.x, program.logit_rows if rows else None,
                        program.R if rows else program.N, self.size, float(self.eps), STREAM], when)
        program.pending = None


register_part("norm", "rmsnorm", RMSNorm)
