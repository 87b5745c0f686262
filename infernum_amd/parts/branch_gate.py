"""A gate on a sublayer's result (category ``branch_gate``).

``sigmoid_linear``: the result is multiplied element by element by sigmoid(G a + b), with a the rows that the sublayer
itself read, G a [width, width] matrix and b a bias.  The part makes the logits G a (fp32 sums, kept in fp32); the
sigmoid, the bias and the product are done by the kernel that takes the sublayer's result next (the norm on the
branch, ``kernels.api.gated_norm_add``), so the gated result is never stored.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Part, Runtime, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights


class SigmoidLinearGate(Part):
    category = "branch_gate"
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, name: str = "weight", bias_name: Optional[str] = "bias",
                 init_std: float = 0.02):
        super().__init__(rt)
        self.hidden_size, self.name, self.bias_name, self.init_std = int(hidden_size), str(name), bias_name, init_std
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        H = self.hidden_size
        out = {self.name: WeightSpec((H, H), ("normal", self.init_std))}
        if self.bias_name is not None:
            out[self.bias_name] = WeightSpec((H,), ("normal", 0.5), follows_compute_dtype=False)
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name].contiguous()
        self.bias = tensors[self.bias_name].to(torch.float32).contiguous() if self.bias_name is not None else None
        prepare_weights(self.rt, [(self.weight, None, True), (self.weight, None, False)])

    # up to so many rows the product's partial sums go on as they are (the kernel that takes the sigmoid adds them: a
    # launch less a branch in steps of single tokens); above, the product leaves one matrix (a third of the bytes
    # for that kernel to read where a long portion's product would be split)
    SPLIT_UP_TO = 128

    def logits(self, a: torch.Tensor):
        """a [N, H] in the compute dtype -> G a, fp32 [N, H] or the partial sums of a split product (the kernel that
        takes the sigmoid adds them, and the bias)."""
        return linear(a, self.weight, out_dtype=torch.float32, keep_split=a.shape[0] <= self.SPLIT_UP_TO,
                      kernels=self.rt.kernels)

    def emit_logits(self, program, key: str):
        """The launches of :meth:`logits` on ``program.x``; returns the Value [N, H] fp32, whole or in parts."""
        from ..engine.program import Guard, Value
        few = Guard.between(program.N, 0, self.SPLIT_UP_TO)
        a = emit_linear(program, program.x, program.N, self.weight, torch.float32, None, True, key, key, when=few)
        b = emit_linear(program, program.x, program.N, self.weight, torch.float32, None, False, key + ".whole",
                        key + ".whole", when=~few)
        return Value(self.hidden_size, list(a.alts) + list(b.alts))


register_part("branch_gate", "sigmoid_linear", SigmoidLinearGate)
