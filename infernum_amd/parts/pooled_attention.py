"""Attention over a sliding window of single keys and, before the window, whole blocks of keys seen through their
means.

q = Wq x + bq, k = Wk x + bk, v = Wv x + bv (the biases optional), heads of ``head_dim`` query/key values and
``value_dim`` values, query head h over key/value head h // (nh / nkv).  The first ``rotary_dim`` values of every q
and k head are rotated (halves), then (``qk_unit_norm``) every q and k head is divided by its root mean square.  A
query at position p sees the keys p - window + 1 .. p one by one and, with ``pool`` P, every block of P positions
b P .. b P + P - 1 that ends at or before p - window as ONE key and value: the means of the block's keys (as the
pages hold them, normed and rotated) and of its values.  Positions that have left the window while their block is
still open are not seen.  Keys and blocks share one softmax; then the output projection.  Without a window every
earlier key is seen and nothing is pooled.

What it keeps: the keys and values of the positions that the window or the open block still need (a ``window``
group of pages whose reach is max(window, P): older pages go back to the pool), and the blocks' means in pages of
a ``full`` group with one entry per P positions (``cached_companions``: a second cached thing with block tables of
its own).  A block's means are made in the step that brings the block's last token, from the pages.  In bfloat16,
head sizes in multiples of 16 up to 256 run on the matrix cores (a kernel for single tokens, whose sixteen columns
are the query heads of a key/value head, and one for portions of prompts); other sizes and the 32-bit path take the
plain kernel, a wave a token and head.
"""
from __future__ import annotations

from typing import Any, Dict, Mapping, Optional, Sequence

import torch

from ..kernels import api as K
from .base import (CacheSpec, CacheView, Mixer, PageTensor, PartSpec, Runtime, StepContext, WeightSpec, make_part,
                   register_part)
from .linear import emit_linear, linear, prepare_weights


class _PooledBlocks:
    """What the mixer keeps per block of positions: not a part of its own (no tensors, no forward), only the
    cache's view of it."""

    def __init__(self, nkv: int, d: int, dv: int, pool: int):
        self.nkv, self.d, self.dv, self.pool = nkv, d, dv, pool

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("full", payload=(PageTensor("pk", (self.nkv, self.d), token_axis=1, every=self.pool),
                                          PageTensor("pv", (self.nkv, self.dv), token_axis=1, every=self.pool)))

    def state_spec(self):
        return None


class PooledWindowAttention(Mixer):
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 scale: float, position: Optional[Mapping[str, Any]] = None, window: Optional[int] = None,
                 pool: Optional[int] = None, bias: bool = True, qk_unit_norm: bool = True, norm_eps: float = 1e-6,
                 init_std: float = 0.02, names: Sequence[str] = ("q", "k", "v", "o")):
        super().__init__(rt)
        if num_heads % num_kv_heads:
            raise ValueError(f"num_heads {num_heads} is not a multiple of num_kv_heads {num_kv_heads}")
        self.hidden_size, self.nh, self.nkv = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.d, self.dv = int(head_dim), int(value_dim)
        if max(self.d, self.dv) > K.WPA_MAX_HEAD_DIM:
            raise ValueError(f"head sizes {self.d}, {self.dv}: at most {K.WPA_MAX_HEAD_DIM}")
        self.scale = float(scale)
        self.window = int(window) if window else 0
        self.pool = int(pool) if (pool and self.window) else 0
        self.bias, self.unit_norm, self.norm_eps = bool(bias), bool(qk_unit_norm), float(norm_eps)
        self.init_std, self.names = init_std, tuple(names)
        pos_spec = PartSpec(**position) if isinstance(position, Mapping) else (position or PartSpec("none"))
        self.position = make_part("position", pos_spec, rt)
        if getattr(self.position, "pairing", "half") != "half" or getattr(self.position, "magnitude", 1.0) != 1.0:
            raise ValueError("this mixer rotates halves, without a factor on sine and cosine")
        self.blocks = _PooledBlocks(self.nkv, self.d, self.dv, self.pool) if self.pool else None
        self.row = (self.nh + self.nkv) * self.d + self.nkv * self.dv
        # bf16 steps run on the matrix cores where the head sizes have a library; otherwise, and in 32-bit, on the
        # plain kernel (a wave a token and head)
        self.use_mfma = (rt.kernels == "auto" and rt.dtype == torch.bfloat16 and rt.device.type == "cuda"
                         and K.wpa_mfma_available(self.d, self.dv))
        self.w_qkv: Optional[torch.Tensor] = None
        self.b_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    # ---- what it needs ---------------------------------------------------
    def cache_spec(self) -> CacheSpec:
        # values transposed within a page, as the second product of the matrix cores reads them
        payload = (PageTensor("k", (self.nkv, self.d), token_axis=1), PageTensor("v", (self.nkv, self.dv), token_axis=2))
        if not self.window:
            return CacheSpec("full", payload=payload)
        # a page is needed while the window reaches it, or the block that is still open
        return CacheSpec("window", window=max(self.window, self.pool), payload=payload)

    def cached_companions(self) -> Dict[str, Any]:
        return {"blocks": self.blocks} if self.blocks is not None else {}

    def step_needs(self) -> Dict[str, Any]:
        return {"row_tiles": K.PREFILL_TILE_ROWS} if self.use_mfma else {}

    def weights(self) -> Dict[str, WeightSpec]:
        nh, nkv, d, dv, H = self.nh, self.nkv, self.d, self.dv, self.hidden_size
        q, k, v, o = self.names
        init = ("normal", self.init_std)
        out = {q: WeightSpec((nh * d, H), init), k: WeightSpec((nkv * d, H), init), v: WeightSpec((nkv * dv, H), init),
               o: WeightSpec((H, nh * dv), init)}
        if self.bias:
            for name, rows in ((q, nh * d), (k, nkv * d), (v, nkv * dv)):
                out[name + ".b"] = WeightSpec((rows,), ("normal", 0.5), follows_compute_dtype=False)
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        q, k, v, o = self.names
        self.w_qkv = torch.cat([tensors[q], tensors[k], tensors[v]], dim=0).contiguous()
        if self.bias:
            self.b_qkv = torch.cat([tensors[n + ".b"].to(torch.float32) for n in (q, k, v)]).contiguous()
        self.w_o = tensors[o].contiguous()
        prepare_weights(self.rt, [(self.w_qkv, None, False), (self.w_o, None, True)])

    def _views(self, cache: CacheView):
        if cache is None or cache.pages.get("k") is None or cache.pages.get("v") is None:
            raise K.KernelError("attention needs pages of the cache")
        if not cache.writable:
            raise K.KernelError("this mixer writes its own pages")
        blocks = cache.others.get("blocks") if self.blocks is not None else None
        if self.blocks is not None and (blocks is None or "pk" not in blocks.pages):
            raise K.KernelError("this mixer needs pages for its blocks' means")
        return cache.pages["k"], cache.pages["v"], blocks

    # ---- one step --------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: CacheView):
        nh, nkv, d, dv = self.nh, self.nkv, self.d, self.dv
        kp, vp, blocks = self._views(cache)
        n, g = x.shape[0], cache.group
        proj = linear(x, self.w_qkv, kernels=self.rt.kernels)
        q = torch.empty((n, nh * d), dtype=x.dtype, device=x.device)
        K.wpa_prepare(proj, self.b_qkv, q, ctx.positions, ctx.slots[g], self.position.inv_freq, self.position.rotary_dim,
                      self.unit_norm, self.norm_eps, kp, vp, nh, nkv, d, dv)
        pk = pv = bt_pool = None
        if blocks is not None:
            pk, pv, bt_pool = blocks.pages["pk"], blocks.pages["pv"], ctx.block_tables[blocks.group]
            K.wpa_pool(kp, vp, pk, pv, ctx.token_seq, ctx.positions, ctx.block_tables[g], bt_pool, self.pool)
        out = torch.empty((n, nh * dv), dtype=x.dtype, device=x.device)
        bt = ctx.block_tables[g]
        if self.use_mfma and kp.shape[2] % 4 == 0:
            nd = ctx.num_decode
            if nd > 0:
                K.wpa_decode(q[:nd], kp, vp, pk, pv, out[:nd], None, ctx.positions[:nd], bt, bt_pool, nh, nkv, self.scale,
                             self.window, self.pool)
            if ctx.num_seqs > nd:
                tiles, num_tiles = ctx.row_tiles(K.PREFILL_TILE_ROWS)
                K.wpa_prefill(q, kp, vp, pk, pv, out, None, ctx.seq_starts, ctx.seq_ctx, bt, bt_pool, tiles, num_tiles,
                              nh, nkv, self.scale, self.window, self.pool)
        else:
            K.wpa_attention(q, kp, vp, pk, pv, out, None, ctx.token_seq, ctx.positions, bt, bt_pool, nh, nkv, self.scale,
                            self.window, self.pool)
        return linear(out, self.w_o, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view: CacheView) -> None:
        if type(self).forward is not PooledWindowAttention.forward:
            return super().native(program, view)
        from ..engine.program import STREAM, Guard
        nh, nkv, d, dv, rt = self.nh, self.nkv, self.d, self.dv, self.rt
        kp, vp, blocks = self._views(view)
        g = view.group
        ps, num_pages = int(kp.shape[2]), int(kp.shape[0])
        T, N, act, ab = program.T, program.N, program.act_code, program.act_bytes
        inv_freq = self.position.inv_freq
        rot = self.position.rotary_dim if inv_freq is not None else 0
        f64 = int(inv_freq is not None and inv_freq.dtype == torch.float64)
        program.keep(kp, vp, inv_freq, self.b_qkv)
        proj = emit_linear(program, program.x, N, self.w_qkv, rt.dtype, None, False, "wpa.proj", "wpa.qkv").tensor()
        q = program.buffer("wpa.q", T * nh * d * ab)
        bt, bt_cols = program.block_table(g), program.bt_cols(g)
        program.op("core", "ia_wpa_prepare", [proj, self.row, self.b_qkv, q, nh * d, act, program.positions,
                                              program.slots(g), inv_freq, f64, rot, int(self.unit_norm),
                                              float(self.norm_eps), kp, vp, N, nh, nkv, d, dv, ps, num_pages, STREAM])
        pk = pv = bt_pool = None
        pool_cols, pool_pages = 0, 0
        if blocks is not None:
            pk, pv = blocks.pages["pk"], blocks.pages["pv"]
            program.keep(pk, pv)
            bt_pool, pool_cols, pool_pages = program.block_table(blocks.group), program.bt_cols(blocks.group), int(pk.shape[0])
            program.op("core", "ia_wpa_pool", [kp, vp, pk, pv, act, program.token_seq, program.positions, bt, bt_cols,
                                               bt_pool, pool_cols, N, nkv, d, dv, ps, num_pages, pool_pages, self.pool,
                                               STREAM])
        out = program.buffer("wpa.out", T * nh * dv * ab)
        if self.use_mfma and ps % 4 == 0:
            lib = K._wpa(d, dv)
            tiles, num_tiles = program.row_tiles(K.PREFILL_TILE_ROWS)
            program.op(lib, "ia_wpa_decode", [q, nh * d, kp, vp, pk, pv, out, None, program.positions, bt, bt_cols, bt_pool,
                                              pool_cols, program.ND, nh, nkv, ps, num_pages, pool_pages, float(self.scale),
                                              self.window, self.pool, STREAM], Guard.between(program.ND, 1))
            program.op(lib, "ia_wpa_prefill", [q, nh * d, kp, vp, pk, pv, out, None, program.seq_starts, program.seq_ctx,
                                               bt, bt_cols, bt_pool, pool_cols, tiles, num_tiles, nh, nkv, ps, num_pages,
                                               pool_pages, float(self.scale), self.window, self.pool, STREAM],
                       Guard.between(program.NP, 1))
        else:
            program.op("core", "ia_wpa_attention", [q, nh * d, kp, vp, pk, pv, out, nh * dv, act, None, program.token_seq,
                                                    program.positions, bt, bt_cols, bt_pool, pool_cols, N, nh, nkv, d, dv,
                                                    ps, num_pages, pool_pages, float(self.scale), self.window, self.pool,
                                                    STREAM])
        program.pending = emit_linear(program, out, N, self.w_o, rt.dtype, None, True, "wpa.mix", "wpa.o")


register_part("mixer", "pooled_window_attention", PooledWindowAttention)
