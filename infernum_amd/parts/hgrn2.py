"""HGRN2: a recurrent mixer whose forget gate also decides what is written.

With heads of ``dim`` key channels and ``vdim`` values, q = silu(Wq x), v = Wv x, and per head and channel the
forget gate f = l + (1 - l) sigmoid(Wf x + b) with a learned lower bound l in [0, 1]:

    S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T,        o_t = S_t^T q_t,

a state S of [dim, vdim] that starts at zero.  Each head's o is divided by its root mean square over vdim and
multiplied by a weight that the heads share; the heads, concatenated, are projected back to the model's width.

It is the recurrence of gated linear attention with the decays given and the keys 1 - f, and runs on that mixer's
kernels (token after token for single tokens, tiles of rows side by side for portions of prompts) in their form for
given decays; a request keeps every head's S in one state slot of fp32 values.  The gate's logits leave their
product in fp32; the sigmoid, the bound, 1 - f, the state and the norm are fp32 whatever the activations' type, and
1 - f is made as (1 - l) sigmoid(-(Wf x + b)), not as the difference of an f that rounding has moved to one.
"""
from __future__ import annotations

from typing import Any, Dict, Sequence

import torch

from ..kernels import api as K
from .base import CacheView, Mixer, Runtime, StateSpec, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights


class Hgrn2(Mixer):
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, norm_eps: float,
                 init_std: float = 0.02, names: Sequence[str] = ("q", "f", "f.b", "lower", "v", "norm", "o")):
        super().__init__(rt)
        self.hidden_size, self.nh, self.dim, self.vdim = int(hidden_size), int(num_heads), int(head_dim), int(value_dim)
        self.norm_eps, self.init_std, self.names = float(norm_eps), init_std, tuple(names)
        if len(self.names) != 7:
            raise ValueError("hgrn2: seven tensor names (q, f, f's bias, lower, v, norm, o)")
        self.nq, self.nv = self.nh * self.dim, self.nh * self.vdim
        self.q_col, self.v_col, self.row = 0, self.nq, self.nq + self.nv       # the projected row: q | v

    def state_spec(self) -> StateSpec:
        return StateSpec((K.gla_state_floats(self.nh, self.dim, self.vdim),))

    def step_needs(self) -> Dict[str, Any]:
        return {"row_tiles": K.PREFILL_TILE_ROWS}

    def weights(self) -> Dict[str, WeightSpec]:
        H, small = self.hidden_size, dict(follows_compute_dtype=False)
        q, f, fb, lower, v, norm, o = self.names
        init = ("normal", self.init_std)
        return {q: WeightSpec((self.nq, H), init), f: WeightSpec((self.nq, H), init),
                fb: WeightSpec((self.nq,), ("uniform", -1.0, 3.0), **small),
                lower: WeightSpec((self.nq,), ("uniform", 0.0, 0.9), **small),
                v: WeightSpec((self.nv, H), init), norm: WeightSpec((self.vdim,), ("uniform", 0.8, 1.2), **small),
                o: WeightSpec((H, self.nv), init)}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        q, f, fb, lower, v, norm, o = self.names
        self.w_in = torch.cat([tensors[q], tensors[v]], dim=0).contiguous()
        self.w_f = tensors[f].contiguous()
        self.b_f = tensors[fb].to(torch.float32).contiguous()
        self.lower = tensors[lower].to(torch.float32).contiguous()
        self.w_norm = tensors[norm].to(torch.float32).contiguous()
        self.w_o = tensors[o].contiguous()
        prepare_weights(self.rt, [(self.w_in, None, False), (self.w_f, None, False), (self.w_o, None, True)])

    def _state(self, cache: CacheView) -> torch.Tensor:
        if cache is None or cache.state is None:
            raise K.KernelError("hgrn2 needs a state slot")
        return cache.state

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: CacheView):
        n, dev = x.shape[0], x.device
        state = self._state(cache)
        proj = linear(x, self.w_in, kernels=self.rt.kernels)                            # [n, q | v]
        f = linear(x, self.w_f, out_dtype=torch.float32, kernels=self.rt.kernels)       # the gate's logits, then the gate
        k = K.hgrn2_gates(proj, self.q_col, f, self.b_f, self.lower)
        o = torch.empty((n, self.nv), dtype=torch.float32, device=dev)
        nd = ctx.num_decode
        if nd > 0:
            K.hgrn2_scan(proj, self.q_col, self.v_col, f, k, state, o, ctx.seq_starts[:nd + 1], ctx.state_slots[:nd],
                         self.nh, self.dim, self.vdim)
        if ctx.num_seqs > nd:
            tiles, num_tiles = ctx.row_tiles(K.PREFILL_TILE_ROWS)
            K.hgrn2_chunked(proj, self.q_col, self.v_col, f, k, state, o, ctx.seq_starts, ctx.state_slots, tiles, num_tiles,
                            nd, self.nh, self.dim, self.vdim)
        normed = torch.empty((n, self.nv), dtype=self.rt.dtype, device=dev)
        K.head_norm_gate(o, None, 0, self.w_norm, self.norm_eps, self.nh, self.vdim, normed)
        return linear(normed, self.w_o, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not Hgrn2.forward:
            return super().native(program, view)
        from ..engine.program import STREAM, Guard
        rt, N, T, act, ab = self.rt, program.N, program.T, program.act_code, program.act_bytes
        state = self._state(view)
        program.keep(state, self.b_f, self.lower, self.w_norm)
        proj = emit_linear(program, program.x, N, self.w_in, rt.dtype, None, False, "hgrn2.proj", "hgrn2.in").tensor()
        f = emit_linear(program, program.x, N, self.w_f, torch.float32, None, False, "hgrn2.f", "hgrn2.gate").tensor()
        k = program.buffer("hgrn2.k", T * self.nq * 4)
        program.op("core", "ia_hgrn2_gates", [proj, act, self.row, self.q_col, f, k, self.nq, self.b_f, self.lower, N,
                                              self.nq, STREAM])
        o = program.buffer("hgrn2.o", T * self.nv * 4)
        program.op("core", "ia_hgrn2_scan", [proj, act, self.row, self.q_col, self.v_col, f, k, self.nq, state,
                                             int(state.stride(0)), o, program.seq_starts, program.state_slots,
                                             program.ND, self.nh, self.dim, self.vdim, STREAM],
                   Guard.between(program.ND, 1))
        floats = K.gla_state_floats(self.nh, self.dim, self.vdim)
        most = -(-T // K.PREFILL_TILE_ROWS) + int(state.shape[0])
        records = program.buffer("hgrn2.records", most * floats * 4)
        decay = program.buffer("hgrn2.decay", most * self.nq * 4)
        tiles, num_tiles = program.row_tiles(K.PREFILL_TILE_ROWS)
        program.op("core", "ia_hgrn2_chunked", [proj, act, self.row, self.q_col, self.v_col, f, k, self.nq, state,
                                                int(state.stride(0)), o, program.seq_starts, program.state_slots, tiles,
                                                num_tiles, program.ND, N, records, floats, decay, self.nh, self.dim,
                                                self.vdim, STREAM], Guard.between(program.NP, 1))
        normed = program.buffer("hgrn2.normed", T * self.nv * ab)
        program.op("core", "ia_head_norm_gate", [o, None, act, 0, 0, self.w_norm, normed, N, self.nh, self.vdim,
                                                 float(self.norm_eps), STREAM])
        program.pending = emit_linear(program, normed, N, self.w_o, rt.dtype, None, True, "hgrn2.out", "hgrn2.o_proj")


register_part("mixer", "hgrn2", Hgrn2)
