"""Routed experts: every token's feed-forward is the weighted sum of ``top`` of E small gated feed-forwards.

  z = R x + b            router logits in fp32 (x as the matrix products read it), bias optional
  chosen = the ``top`` largest z (lowest index among equals);  weight = softmax over the chosen z alone
  expert e:  g = min(G_e x, limit),  u = clamp(U_e x, -limit, limit),  y = g sigmoid(alpha g) (u + 1),  D_e y
  out = sum over the chosen, in the order of the choices, of weight * expert(x)

``limit`` and ``alpha`` are parameters (alpha = 1.702 is the sigmoid form of GELU).  The experts' matrices are
kept stacked, [E, 2 ff, W] with the rows of G_e and U_e alternating (so that a gate value and its up value
end in one thread of the product's tile) and [E, W, ff].  The tokens are grouped by expert on the device, and
only the chosen experts' weights are read.  The result is left as fp32 parts [top, N, W], one per choice, each
already times its weight, which the next norm adds in the order of the choices: an expert's output is never
rounded to the compute dtype.

Options for other designs.  ``gated=False``: an expert is D_e act(U_e x) without a gate (``activation`` names the
function: ``relu_squared``, ``gelu``, ``gelu_tanh``; tensors ``e<i>.up`` and ``e<i>.down``).  ``router="softmax_top"``:
s = softmax(z) over ALL experts, the ``top`` largest of s + correction are chosen (``correction``: a stored vector that
moves the choice only), and the weights are the chosen s over their sum (+ 1e-20).  ``shared_ff``: one more expert of
that middle width (``shared.up``, ``shared.down``; same form, no gate) that every token takes with weight 1; its
result is added into the first choice's part.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import api as K
from .base import FeedForward, Runtime, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear


class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, intermediate_size: int, num_experts: int, top: int,
                 limit: Optional[float] = None, alpha: float = 1.702, router_bias: bool = True,
                 router_name: str = "router", expert_prefix: str = "e", init_std: float = 0.02, gated: bool = True,
                 activation: str = "relu_squared", router: str = "top_softmax", correction_name: str = "correction",
                 shared_ff: Optional[int] = None):
        super().__init__(rt)
        self.hidden_size, self.ff = int(hidden_size), int(intermediate_size)
        self.num_experts, self.top = int(num_experts), int(top)
        if not 0 < self.top <= self.num_experts:
            raise ValueError(f"a token takes {top} of {num_experts} experts")
        self.gated, self.activation, self.router = bool(gated), str(activation), str(router)
        if self.router not in ("top_softmax", "softmax_top"):
            raise ValueError(f"router {router!r}: 'top_softmax' or 'softmax_top'")
        if not self.gated and self.activation not in K.ACTIVATIONS:
            raise ValueError(f"activation {activation!r}: one of {sorted(K.ACTIVATIONS)}")
        self.limit, self.alpha = float(limit) if limit is not None else 0.0, float(alpha)
        if self.gated and not self.limit > 0:
            raise ValueError("the experts' limit must be positive")
        self.correction_name = correction_name
        self.shared_ff = int(shared_ff) if shared_ff else 0
        if self.shared_ff and self.gated:
            raise ValueError("a shared expert goes with experts without a gate")
        self.router_bias, self.router_name, self.expert_prefix = bool(router_bias), router_name, expert_prefix
        self.init_std = init_std
        self.w_router: Optional[torch.Tensor] = None
        self.b_router: Optional[torch.Tensor] = None
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def weights(self) -> Dict[str, WeightSpec]:
        H, I, E = self.hidden_size, self.ff, self.num_experts
        init = ("normal", self.init_std)
        out = {self.router_name: WeightSpec((E, H), init)}
        if self.router == "softmax_top":
            out[self.correction_name] = WeightSpec((E,), ("normal", 0.05), follows_compute_dtype=False)
        elif self.router_bias:
            out[self.router_name + ".b"] = WeightSpec((E,), ("normal", 0.5), follows_compute_dtype=False)
        if self.shared_ff:
            out["shared.up"] = WeightSpec((self.shared_ff, H), init)
            out["shared.down"] = WeightSpec((H, self.shared_ff), init)
        for e in range(E):
            p = f"{self.expert_prefix}{e}."
            if self.gated:
                out[p + "gate"] = WeightSpec((I, H), init)
            out[p + "up"] = WeightSpec((I, H), init)
            out[p + "down"] = WeightSpec((H, I), init)
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        H, I, E = self.hidden_size, self.ff, self.num_experts
        self.w_router = tensors[self.router_name].contiguous()
        if self.router == "softmax_top":
            self.b_router = tensors[self.correction_name].contiguous()
        else:
            self.b_router = tensors[self.router_name + ".b"].contiguous() if self.router_bias else None
        dev, dt = self.w_router.device, self.w_router.dtype
        self.w_gate_up = torch.empty((E, (2 if self.gated else 1) * I, H), dtype=dt, device=dev)
        self.w_down = torch.empty((E, H, I), dtype=dt, device=dev)
        for e in range(E):
            p = f"{self.expert_prefix}{e}."
            if self.gated:
                self.w_gate_up[e, 0::2] = tensors[p + "gate"]
                self.w_gate_up[e, 1::2] = tensors[p + "up"]
            else:
                self.w_gate_up[e] = tensors[p + "up"]
            self.w_down[e] = tensors[p + "down"]
        if self.shared_ff:
            from .linear import prepare_weights
            self.w_shared_up, self.w_shared_down = tensors["shared.up"].contiguous(), tensors["shared.down"].contiguous()
            prepare_weights(self.rt, [(self.w_shared_up, None, False), (self.w_shared_down, None, False)])

    def forward(self, x: torch.Tensor, ctx: Optional[StepContext] = None):
        z = linear(x, self.w_router, out_dtype=torch.float32, kernels=self.rt.kernels)
        choose = K.router_softmax_topk if self.router == "softmax_top" else K.router_topk
        ids, weights = choose(z, self.b_router, self.top)
        if self.gated:
            return K.moe_experts(x, ids, weights, self.w_gate_up, self.w_down, self.limit, self.alpha)
        parts = K.moe_plain_experts(x, ids, weights, self.w_gate_up, self.w_down, self.activation)
        if self.shared_ff:
            u = K.activation(linear(x, self.w_shared_up, kernels=self.rt.kernels), self.activation)
            K.stream_add(parts[0], linear(u, self.w_shared_down, out_dtype=torch.float32, kernels=self.rt.kernels))
        return K.SplitSum(parts)

    def native(self, program, view=None) -> None:
        if type(self).forward is not RoutedExperts.forward:
            return super().native(program, view)
        from ..engine.program import ALWAYS, STREAM, Alt, Value
        H, I, E, top, T, N = self.hidden_size, self.ff, self.num_experts, self.top, program.T, program.N
        program.keep(self.w_router, self.b_router, self.w_gate_up, self.w_down)
        z = emit_linear(program, program.x, N, self.w_router, torch.float32, None, False, "moe.logits", "moe.router")
        ids = program.buffer("moe.ids", T * top * 4)
        wts = program.buffer("moe.weights", T * top * 4)
        offsets = program.buffer("moe.offsets", (E + 1) * 4)
        perm = program.buffer("moe.perm", T * top * 4)
        y = program.buffer("moe.y", T * top * I * program.act_bytes)
        parts = program.buffer("moe.parts", top * T * H * 4)
        b = self.b_router
        choose = "ia_router_softmax_topk" if self.router == "softmax_top" else "ia_router_topk"
        program.op("core", choose, [z.tensor(), b, K.DTYPE_CODE[b.dtype] if b is not None else 0, ids, wts,
                                    N, E, top, STREAM])
        program.op("core", "ia_moe_sort", [ids, offsets, perm, N * top, E, STREAM])
        if not self.gated:
            return self._native_plain(program, ids, wts, offsets, perm, y, parts)
        from ..engine.program import NEVER, Guard
        first = K.moe_grouped_from_tokens(E, top, H, I, self.rt.dtype)
        grouped = Guard.between(N, first) if first > 0 else NEVER
        tiled = ~grouped
        program.op("core", "ia_moe_gate_up", [program.x, self.w_gate_up, y, offsets, perm, program.act_code, N * top,
                                              E, top, H, I, self.limit, self.alpha, STREAM], tiled)
        program.op("core", "ia_moe_down", [y, self.w_down, parts, wts, offsets, perm, program.act_code, N, E, top, H,
                                           I, STREAM], tiled)
        if first > 0 and first <= T:
            # steps of many tokens: the grouped form of the LDS-tiled product (kernels.api.moe_experts)
            xs = program.buffer("moe.sorted", T * top * H * program.act_bytes)
            gu = program.buffer("moe.gate_up", T * top * 2 * I * program.act_bytes)
            program.op("core", "ia_moe_gather", [program.x, perm, xs, N * top, top, H, STREAM], grouped)
            program.op("core", "ia_gemm_mfma_grouped", [xs, self.w_gate_up, gu, offsets, E, N * top, 2 * I, H, STREAM],
                       grouped)
            program.op("core", "ia_moe_glu", [gu, y, N * top, I, self.limit, self.alpha, STREAM], grouped)
            program.op("core", "ia_gemm_mfma_grouped", [y, self.w_down, xs, offsets, E, N * top, H, I, STREAM], grouped)
            program.op("core", "ia_moe_scatter", [xs, perm, wts, parts, N, top, H, STREAM], grouped)
        program.pending = Value(H, [Alt(ALWAYS, parts, top, torch.float32)])


    def _native_plain(self, program, ids, wts, offsets, perm, y, parts) -> None:
        """The launches of ``kernels.api.moe_plain_experts`` and of the shared expert."""
        from ..engine.program import ALWAYS, NEVER, STREAM, Alt, Guard, Value
        from .linear import emit_linear as emit
        H, I, E, top, T, N = self.hidden_size, self.ff, self.num_experts, self.top, program.T, program.N
        act, code = K.ACTIVATIONS[self.activation], program.act_code
        first = K.moe_grouped_from_tokens(E, top, H, I, self.rt.dtype)
        grouped = Guard.between(N, first) if 0 < first <= T else NEVER
        tiled = ~grouped
        program.op("core", "ia_moe_up", [program.x, self.w_gate_up, y, offsets, perm, code, N * top, E, top, H, I, act,
                                         STREAM], tiled)
        program.op("core", "ia_moe_down", [y, self.w_down, parts, wts, offsets, perm, code, N, E, top, H, I, STREAM],
                   tiled)
        if 0 < first <= T:
            xs = program.buffer("moe.sorted", T * top * H * program.act_bytes)
            program.op("core", "ia_moe_gather", [program.x, perm, xs, N * top, top, H, STREAM], grouped)
            program.op("core", "ia_gemm_mfma_grouped", [xs, self.w_gate_up, y, offsets, E, N * top, I, H, STREAM], grouped)
            program.op("core", "ia_activation", [y, y, code, N * (top * I), act, STREAM], grouped)
            program.op("core", "ia_gemm_mfma_grouped", [y, self.w_down, xs, offsets, E, N * top, H, I, STREAM], grouped)
            program.op("core", "ia_moe_scatter", [xs, perm, wts, parts, N, top, H, STREAM], grouped)
        if self.shared_ff:
            program.keep(self.w_shared_up, self.w_shared_down)
            u = emit(program, program.x, N, self.w_shared_up, self.rt.dtype, None, False, "moe.shared.act",
                     "moe.shared.up").tensor()
            program.op("core", "ia_activation", [u, u, code, N * self.shared_ff, act, STREAM])
            down = emit(program, u, N, self.w_shared_down, torch.float32, None, True, "moe.shared.out", "moe.shared.down")
            f32 = K.DTYPE_CODE[torch.float32]
            for alt in down.alts:
                program.op("core", "ia_stream_add", [parts, alt.where, f32, alt.splits or 1, N, H, STREAM], alt.when)
        program.pending = Value(H, [Alt(ALWAYS, parts, top, torch.float32)])


register_part("feed_forward", "routed_experts", RoutedExperts)
