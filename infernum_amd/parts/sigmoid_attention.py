"""Attention over the paged cache whose weights are sigmoids, not a softmax.

q = x Wq^T + bq, k = x Wk^T + bk (heads of ``head_dim``), v = x Wv^T + bv (heads of ``value_dim``); all of a token's
queries together are divided by their root mean square and multiplied by a weight per value, and so are all of its
keys; the queries are multiplied by 1 + coef ln(floor((p + 1) / every) + 1) at position p when the mixer has such a
factor.  There is no rotation.  Query head h reads key/value head h // (nh / nkv); for the key at j <= p

    w = sigmoid( scale q.k_j - r1_h ln(1 + r2_h (p - j)) + b_h ),     out_h = sigmoid(gate_h) sum_j w v_j,

with nothing normalised over the keys, r1, r2, b numbers per head and gate = x Wg^T one number per token and head.
Then the output projection.  One product makes q, k, v and the gates' logits; keys are kept [nkv, page, head_dim]
and values transposed, [nkv, value_dim, page], per page.  Scores, the distance term, sigmoids and the sums over the keys are fp32.

In bf16, with head sizes that are multiples of 16 up to 256 and a page size that is a multiple of 4, the two products
run on the matrix cores: one kernel for the step's single tokens (its first rows), one for its portions of prompts;
every other case takes the plain kernel, one wave per token and head.
"""
from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import api as K
from .base import CacheSpec, CacheView, Mixer, PageTensor, Runtime, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights


class SigmoidAttention(Mixer):
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 scale: float, norm_eps: float, q_temp: Optional[Mapping[str, Any]] = None, biases: bool = True,
                 gate: bool = True, distance_bias: bool = True, kernels: str = "auto", init_std: float = 0.02):
        """``q_temp`` {coef, every} or None; ``biases``: q, k and v have them; ``gate``: a sigmoid gate per token and
        head on the output; ``distance_bias``: the heads have r1, r2 (the term r1 ln(1 + r2 distance) taken off the
        score) and the number b added to it."""
        super().__init__(rt)
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        self.hidden_size, self.nh, self.nkv = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dim, self.vdim = int(head_dim), int(value_dim)
        if max(self.dim, self.vdim) > K.GENERIC_MAX_HEAD_DIM:
            raise ValueError(f"head sizes above {K.GENERIC_MAX_HEAD_DIM} have no attention kernel")
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.temp_coef = float(q_temp["coef"]) if q_temp else 0.0
        self.temp_every = int(q_temp["every"]) if q_temp else 0
        self.biases, self.gate, self.distance_bias, self.init_std = bool(biases), bool(gate), bool(distance_bias), init_std
        self.nq, self.nk, self.nv = self.nh * self.dim, self.nkv * self.dim, self.nkv * self.vdim
        self.row = self.nq + self.nk + self.nv + (self.nh if self.gate else 0)
        self.bq = self.bk = self.bv = self.r1 = self.r2 = self.pb = None
        if kernels not in ("auto", "generic"):
            raise ValueError("kernels must be 'auto' or 'generic'")
        self.use_mfma = (kernels == "auto" and rt.kernels == "auto" and rt.dtype == torch.bfloat16
                         and rt.device.type == "cuda" and K.sigattn_mfma_available(self.dim, self.vdim))

    # ---- what it needs ---------------------------------------------------
    def cache_spec(self) -> CacheSpec:
        return CacheSpec("full", payload=(PageTensor("k", (self.nkv, self.dim), token_axis=1),
                                          PageTensor("v", (self.nkv, self.vdim), token_axis=2)))

    def step_needs(self) -> Dict[str, Any]:
        # the matrix-core kernel for portions of prompts works on tiles of 64 query rows
        return {"row_tiles": K.PREFILL_TILE_ROWS} if self.use_mfma else {}

    def weights(self) -> Dict[str, WeightSpec]:
        H, init, small = self.hidden_size, ("normal", self.init_std), dict(follows_compute_dtype=False)
        out = {"q": WeightSpec((self.nq, H), init), "k": WeightSpec((self.nk, H), init), "v": WeightSpec((self.nv, H), init),
               "q.norm": WeightSpec((self.nq,), ("uniform", 0.8, 1.2), **small),
               "k.norm": WeightSpec((self.nk,), ("uniform", 0.8, 1.2), **small),
               "o": WeightSpec((H, self.nh * self.vdim), init)}
        if self.biases:
            out.update({"q.b": WeightSpec((self.nq,), ("normal", 0.1), **small),
                        "k.b": WeightSpec((self.nk,), ("normal", 0.1), **small),
                        "v.b": WeightSpec((self.nv,), ("normal", 0.1), **small)})
        if self.distance_bias:
            out.update({"r1": WeightSpec((self.nh,), ("uniform", 0.2, 1.0), **small),
                        "r2": WeightSpec((self.nh,), ("uniform", 0.05, 0.5), **small),
                        "pb": WeightSpec((self.nh,), ("uniform", -3.0, -1.0), **small)})
        if self.gate:
            out["g"] = WeightSpec((self.nh, H), init)
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()           # noqa: E731
        rows = [tensors["q"], tensors["k"], tensors["v"]] + ([tensors["g"]] if self.gate else [])
        self.w_in = torch.cat(rows, dim=0).contiguous()
        self.w_o = tensors["o"].contiguous()
        self.wq, self.wk = f32("q.norm"), f32("k.norm")
        if self.biases:
            self.bq, self.bk, self.bv = f32("q.b"), f32("k.b"), f32("v.b")
        if self.distance_bias:
            self.r1, self.r2, self.pb = f32("r1"), f32("r2"), f32("pb")
        prepare_weights(self.rt, [(self.w_in, None, False), (self.w_in[: self.nq], None, False), (self.w_o, None, True)])

    # ---- one step --------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: CacheView):
        if cache.k_pages is None or cache.v_pages is None:
            raise K.KernelError("attention needs pages of the cache")
        if not cache.writable:
            raise K.KernelError("sigmoid_attention: every run writes its own keys and values")
        n, g = x.shape[0], cache.group
        proj = linear(x, self.w_in, kernels=self.rt.kernels)                     # [n, q | k | v | gate logits]
        q = torch.empty((n, self.nq), dtype=self.rt.dtype, device=x.device)
        K.sigattn_prepare(proj, self.bq, self.bk, self.bv, self.wq, self.wk, self.norm_eps, self.temp_coef,
                          self.temp_every, ctx.positions, ctx.slots[g], q, cache.k_pages, cache.v_pages, self.nh,
                          self.nkv, self.dim, self.vdim)
        out = torch.empty((n, self.nh * self.vdim), dtype=self.rt.dtype, device=x.device)
        gate = proj[:, self.nq + self.nk + self.nv:] if self.gate else None
        self.attend(q, gate, out, ctx, cache)
        return linear(out, self.w_o, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not SigmoidAttention.forward or type(self).attend is not SigmoidAttention.attend:
            return super().native(program, view)
        from ..engine.program import STREAM
        if view.k_pages is None or view.v_pages is None or not view.writable:
            raise K.KernelError("sigmoid_attention: every run needs pages of its own")
        rt, N, T, act, ab = self.rt, program.N, program.T, program.act_code, program.act_bytes
        k, v, g = view.k_pages, view.v_pages, view.group
        ps, num_pages = int(k.shape[2]), int(k.shape[0])
        program.keep(k, v, self.bq, self.bk, self.bv, self.wq, self.wk, self.r1, self.r2, self.pb)
        proj = emit_linear(program, program.x, N, self.w_in, rt.dtype, None, False, "sigattn.proj", "sigattn.in").tensor()
        q = program.buffer("sigattn.q", T * self.nq * ab)
        program.op("core", "ia_sigattn_prepare", [proj, act, self.row, self.bq, self.bk, self.bv, self.wq, self.wk,
                                                  float(self.norm_eps), float(self.temp_coef), int(self.temp_every),
                                                  program.positions, program.slots(g), q, k, v, N, self.nh, self.nkv,
                                                  self.dim, self.vdim, ps, num_pages, STREAM])
        out = program.buffer("sigattn.out", T * self.nh * self.vdim * ab)
        gate = proj.at((self.nq + self.nk + self.nv) * ab) if self.gate else None
        self.emit_attend(program, view, q, gate, out)
        program.pending = emit_linear(program, out, N, self.w_o, rt.dtype, None, True, "sigattn.o", "sigattn.o_proj")

    def emit_attend(self, program, view: CacheView, q, gate, out) -> None:
        from ..engine.program import STREAM, Guard
        k, v, g = view.k_pages, view.v_pages, view.group
        ps, num_pages = int(k.shape[2]), int(k.shape[0])
        gate_stride = self.row if gate is not None else 0
        bt, bt_cols = program.block_table(g), program.bt_cols(g)
        if not (self.use_mfma and ps % 4 == 0):
            program.op("core", "ia_sigattn_generic", [q, self.nq, k, v, gate, gate_stride, out, program.act_code,
                                                      program.token_seq, program.positions, bt, bt_cols, self.r1, self.r2,
                                                      self.pb, program.N, self.nh, self.nkv, self.dim, self.vdim, ps,
                                                      num_pages, float(self.scale), STREAM])
            return
        lib = K._sigattn(self.dim, self.vdim)
        records = program.T + 1024          # tokens x parts of their keys: what fills the GPU, or the tokens themselves
        part = program.buffer("sigattn.part", records * self.nh * self.vdim * 4)
        nh, nkv, dev = self.nh, self.nkv, self.rt.device

        def parts_of_the_keys(ctx: StepContext) -> int:
            nd = ctx.num_decode
            if nd == 0:
                return 1
            if ctx.block_tables[g].shape[1] * ps < ctx.max_total_len:
                raise K.KernelError("sigmoid_attention: the block tables are narrower than the longest request")
            n = K.sigattn_decode_parts(nd, nh, nkv, ctx.max_total_len, dev)
            return max(1, min(n, records // nd))
        parts = program.scalar(("sigmoid_attention: parts of the keys", nh, nkv, g, ps), parts_of_the_keys)
        tiles, num_tiles = program.row_tiles(K.PREFILL_TILE_ROWS)
        program.op(lib, "ia_sigattn_decode", [q, self.nq, k, v, gate, gate_stride, out, part, program.positions, bt,
                                              bt_cols, self.r1, self.r2, self.pb, program.ND, nh, nkv, ps, num_pages,
                                              float(self.scale), parts, STREAM], Guard.between(program.ND, 1))
        program.op(lib, "ia_sigattn_prefill", [q, self.nq, k, v, gate, gate_stride, out, program.seq_starts,
                                               program.seq_ctx, bt, bt_cols, tiles, num_tiles, self.r1, self.r2, self.pb,
                                               nh, nkv, ps, num_pages, float(self.scale), STREAM],
                   Guard.between(program.NP, 1))

    def attend(self, q: torch.Tensor, gate: Optional[torch.Tensor], out: torch.Tensor, ctx: StepContext,
               cache: CacheView) -> None:
        bt = ctx.block_tables[cache.group]
        if not (self.use_mfma and cache.k_pages.shape[2] % 4 == 0):
            K.sigattn_generic(q, cache.k_pages, cache.v_pages, gate, out, ctx.token_seq, ctx.positions, bt, self.r1,
                              self.r2, self.pb, self.nh, self.nkv, self.dim, self.vdim, self.scale)
            return
        nd = ctx.num_decode
        if nd > 0:
            K.sigattn_decode(q[:nd], cache.k_pages, cache.v_pages, gate[:nd] if gate is not None else None, out[:nd],
                             ctx.positions[:nd], bt, self.r1, self.r2, self.pb, self.nh, self.nkv, self.dim, self.vdim,
                             self.scale, ctx.max_total_len)
        if ctx.num_seqs > nd:
            tiles, num_tiles = ctx.row_tiles(K.PREFILL_TILE_ROWS)
            K.sigattn_prefill(q, cache.k_pages, cache.v_pages, gate, out, ctx.seq_starts, ctx.seq_ctx, bt, tiles,
                              num_tiles, self.r1, self.r2, self.pb, self.nh, self.nkv, self.dim, self.vdim, self.scale)


register_part("mixer", "sigmoid_attention", SigmoidAttention)
