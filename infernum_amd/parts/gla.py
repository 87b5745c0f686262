"""Gated linear attention: a recurrent mixer with one decay per key channel and token.

One input projection makes, side by side in a row, q and k (heads x dim each), v and the output gate g (heads x vdim
each); the decay's logits z (heads x dim, fp32) come through a narrow middle, two small products.
Per head, with alpha = sigmoid(z + b)^(1/tau) and a state S of [dim, vdim] that starts at zero:

    S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,        o_t = S_t^T (dim^(-1/2) q_t).

Each head's o is divided by its root mean square over vdim, multiplied by a weight that the heads share and by
silu(g), and the heads, concatenated, are projected back to the model's width.

Between steps a request keeps every head's S in one state slot of fp32 values (in the slices the kernel works on:
``kernels.api.gla_state_floats``).  Decays, their logarithms, the state and the norm are fp32 whatever the
activations' type.
"""
from __future__ import annotations

from typing import Any, Dict, Optional, Sequence

import torch

from ..kernels import api as K
from .base import CacheView, Mixer, Runtime, StateSpec, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights


class GatedLinearAttention(Mixer):
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, tau: float,
                 decay_rank: Optional[int], norm_eps: float, q_scale: Optional[float] = None, init_std: float = 0.02,
                 names: Sequence[str] = ("q", "k", "v", "g", "a1", "a2", "a2.b", "norm", "o")):
        """``decay_rank``: the width of the decay logits' middle (None: read off the tensors of a file).  ``q_scale``: the factor on the queries (default
        head_dim^(-1/2)).  ``names``: the local names of the tensors, in the order of the default."""
        super().__init__(rt)
        self.hidden_size, self.nh, self.dim, self.vdim = int(hidden_size), int(num_heads), int(head_dim), int(value_dim)
        self.tau, self.norm_eps = float(tau), float(norm_eps)
        self.rank = int(decay_rank) if decay_rank else -1
        if not self.tau > 0:
            raise ValueError(f"tau must be positive, got {tau}")
        self.q_scale = float(q_scale) if q_scale is not None else self.dim ** -0.5
        self.init_std, self.names = init_std, tuple(names)
        if len(self.names) != 9:
            raise ValueError("gla: nine tensor names (q, k, v, g, a1, a2, a2's bias, norm, o)")
        nq, nv = self.nh * self.dim, self.nh * self.vdim
        # columns of the projected row: q | k | v | g
        self.q_col, self.k_col, self.v_col, self.g_col = 0, nq, 2 * nq, 2 * nq + nv
        self.row = 2 * nq + 2 * nv

    # ---- what it needs ---------------------------------------------------
    def state_spec(self) -> StateSpec:
        return StateSpec((K.gla_state_floats(self.nh, self.dim, self.vdim),))

    def weights(self) -> Dict[str, WeightSpec]:
        H, nq, nv, small = self.hidden_size, self.nh * self.dim, self.nh * self.vdim, dict(follows_compute_dtype=False)
        q, k, v, g, a1, a2, a2b, norm, o = self.names
        init = ("normal", self.init_std)
        return {q: WeightSpec((nq, H), init), k: WeightSpec((nq, H), init), v: WeightSpec((nv, H), init),
                g: WeightSpec((nv, H), init), a1: WeightSpec((self.rank, H), init),
                a2: WeightSpec((nq, self.rank), ("normal", max(self.rank, 1) ** -0.5)),
                a2b: WeightSpec((nq,), ("uniform", 1.0, 4.0), **small),
                norm: WeightSpec((self.vdim,), ("uniform", 0.8, 1.2), **small), o: WeightSpec((H, nv), init)}

    def step_needs(self) -> Dict[str, Any]:
        # portions of prompts run as tiles of rows side by side
        return {"row_tiles": K.PREFILL_TILE_ROWS}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        q, k, v, g, a1, a2, a2b, norm, o = self.names
        self.w_in = torch.cat([tensors[q], tensors[k], tensors[v], tensors[g]], dim=0).contiguous()
        self.w_a1, self.w_a2 = tensors[a1].contiguous(), tensors[a2].contiguous()
        if self.w_a1.shape[0] != self.w_a2.shape[1]:
            raise ValueError(f"gla: the decay's two matrices do not meet: {tuple(self.w_a1.shape)} and {tuple(self.w_a2.shape)}")
        self.b_a2 = tensors[a2b].to(torch.float32).contiguous()
        self.w_norm = tensors[norm].to(torch.float32).contiguous()
        self.w_o = tensors[o].contiguous()
        prepare_weights(self.rt, [(self.w_in, None, False), (self.w_o, None, True)])

    def _state(self, cache: CacheView) -> torch.Tensor:
        if cache is None or cache.state is None:
            raise K.KernelError("gla needs a state slot")
        return cache.state

    # ---- one step --------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: CacheView):
        n, dev, nv = x.shape[0], x.device, self.nh * self.vdim
        state = self._state(cache)
        proj = linear(x, self.w_in, kernels=self.rt.kernels)                    # [n, q | k | v | g]
        mid = linear(x, self.w_a1, kernels=self.rt.kernels)
        z = linear(mid, self.w_a2, out_dtype=torch.float32, kernels=self.rt.kernels)
        o = torch.empty((n, nv), dtype=torch.float32, device=dev)
        nd = ctx.num_decode
        if nd > 0:          # single tokens: the recurrence itself, a workgroup per request, head and slice of the state
            K.gla_scan(proj, self.q_col, self.k_col, self.v_col, z, self.b_a2, self.tau, self.q_scale, state, o,
                       ctx.seq_starts[:nd + 1], ctx.state_slots[:nd], self.nh, self.dim, self.vdim)
        if ctx.num_seqs > nd:          # portions of prompts: tiles of rows side by side
            tiles, num_tiles = ctx.row_tiles(K.PREFILL_TILE_ROWS)
            K.gla_chunked(proj, self.q_col, self.k_col, self.v_col, z, self.b_a2, self.tau, self.q_scale, state, o,
                          ctx.seq_starts, ctx.state_slots, tiles, num_tiles, nd, self.nh, self.dim, self.vdim)
        gated = torch.empty((n, nv), dtype=self.rt.dtype, device=dev)
        K.head_norm_gate(o, proj, self.g_col, self.w_norm, self.norm_eps, self.nh, self.vdim, gated)
        return linear(gated, self.w_o, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not GatedLinearAttention.forward:
            return super().native(program, view)
        from ..engine.program import STREAM
        rt, N, T, act, ab = self.rt, program.N, program.T, program.act_code, program.act_bytes
        nq, nv = self.nh * self.dim, self.nh * self.vdim
        state = self._state(view)
        program.keep(state, self.b_a2, self.w_norm)
        proj = emit_linear(program, program.x, N, self.w_in, rt.dtype, None, False, "gla.proj", "gla.in").tensor()
        mid = emit_linear(program, program.x, N, self.w_a1, rt.dtype, None, False, "gla.mid", "gla.a1").tensor()
        z = emit_linear(program, mid, N, self.w_a2, torch.float32, None, False, "gla.z", "gla.a2").tensor()
        o = program.buffer("gla.o", T * nv * 4)
        from ..engine.program import Guard
        program.op("core", "ia_gla_scan", [proj, act, self.row, self.q_col, self.k_col, self.v_col, z, nq, self.b_a2,
                                           float(self.tau), float(self.q_scale), state, int(state.stride(0)), o,
                                           program.seq_starts, program.state_slots, program.ND, self.nh, self.dim,
                                           self.vdim, STREAM], Guard.between(program.ND, 1))
        # a request holds a state slot, and a tile at least one row: so many tiles a step has at most
        floats = K.gla_state_floats(self.nh, self.dim, self.vdim)
        most = -(-T // K.PREFILL_TILE_ROWS) + int(state.shape[0])
        records = program.buffer("gla.records", most * floats * 4)
        decay = program.buffer("gla.decay", most * nq * 4)
        tiles, num_tiles = program.row_tiles(K.PREFILL_TILE_ROWS)
        program.op("core", "ia_gla_chunked", [proj, act, self.row, self.q_col, self.k_col, self.v_col, z, nq, self.b_a2,
                                              float(self.tau), float(self.q_scale), state, int(state.stride(0)), o,
                                              program.seq_starts, program.state_slots, tiles, num_tiles, program.ND, N, records,
                                              floats,
                                              decay, self.nh, self.dim, self.vdim, STREAM], Guard.between(program.NP, 1))
        gated = program.buffer("gla.gated", T * nv * ab)
        program.op("core", "ia_head_norm_gate", [o, proj, act, self.row, self.g_col, self.w_norm, gated, N, self.nh,
                                                 self.vdim, float(self.norm_eps), STREAM])
        program.pending = emit_linear(program, gated, N, self.w_o, rt.dtype, None, True, "gla.out", "gla.o_proj")


register_part("mixer", "gla", GatedLinearAttention)
