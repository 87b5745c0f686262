"""Latent attention: the keys and values of all heads come from one low-rank latent per token.

With H heads, per head ``dim`` plain and ``rot_dim`` rotated query/key values, value size ``value_dim`` and latent
size ``rank``:

  q        = Wq x                      [H, dim | rot_dim]
  (l, r)   = Wdkv x                    l [rank], r [rot_dim]: one rotated key part for all heads
  c        = RMSNorm(l) * w_c          the latent
  k_h      = (Uk_h c | rope(r)),   v_h = Uv_h c,   score_h(i, j) = scale * q_h(i) . k_h(j)
  out      = Wo ( concat_h(softmax_h V) * sigmoid(Wg x) )        (the gate is optional)

Only c and rope(r) are cached.  Since q_plain_h . (Uk_h c) = (Uk_h^T q_plain_h) . c, every head's query becomes
one vector (rope(q_rot_h) | Uk_h^T q_plain_h) against the one cached key (rope(r) | c), and the attended value
is the latent itself, to which Uv_h is applied afterwards: this is attention with H query heads over ONE key/value
head of size rot_dim + rank, and it runs on the attention mixer's own rotation, page write and attention kernels
(prefill, decode, fused decode, window and all), which this part inherits.  The rotated values stand first in
that head, where those kernels rotate.  Around them: one product for Wq, Wdkv and Wg together, a kernel that
normalises the latent and lays the rows out, and a product per head for Uk^T and for Uv (with the gate in its
epilogue).

Options: ``q_rank`` (the queries come through a latent of their own, q = Wuq RMSNorm(Wdq x) * w_q, in place of
Wq x); ``sink`` (a learned number per head whose exponential is added to the head's softmax denominator; it has no
key and no value); a position encoding that pairs neighbouring values (the rows of the rotated parts are then kept
in the order in which the kernels' half-split pairs are those pairs).

Pages: keys [num_pages, 1, page_size, rot_dim + rank] and, for the kernels' P.V product, the same latents
transposed, [num_pages, 1, rot_dim + rank, page_size] (zeros in the rot_dim rows).
"""
from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from ..kernels import api as K
from .attention import Attention
from .base import CacheView, Runtime, StepContext, WeightSpec, register_part
from .linear import emit_linear, linear, prepare_weights


class LatentAttention(Attention):
    graph_safe = True

    def __init__(self, rt: Runtime, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int,
                 rank: int, norm_eps: float, scale: float, position: Optional[Mapping[str, Any]] = None,
                 window: Optional[int] = None, gate: bool = True, kernels: str = "auto", init_std: float = 0.02,
                 names: Optional[Mapping[str, str]] = None, q_rank: Optional[int] = None, sink: bool = False):
        self.dn, self.dr, self.dv, self.rank = int(head_dim), int(rot_dim), int(value_dim), int(rank)
        if min(self.dn, self.dv, self.rank) <= 0 or self.dr < 0:
            raise ValueError("latent attention: head sizes and the latent's size must be positive")
        super().__init__(rt, hidden_size, num_heads, 1, self.dr + self.rank, position=position, window=window,
                         scale=scale, kernels=kernels, init_std=init_std)
        if self.position.rotary_dim > self.dr:
            raise ValueError(f"latent attention: {self.position.rotary_dim} rotated values, but the rotated part has {self.dr}")
        self.norm_eps, self.gate = float(norm_eps), bool(gate)
        self.q_rank, self.sink = (int(q_rank) if q_rank else 0), bool(sink)
        self.names = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "g": "g", "o": "o",
                      "dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "sink": "sink"}
        self.names.update(names or {})
        self.w_uq: Optional[torch.Tensor] = None            # [H (dn + dr), q_rank] when the queries have a latent
        self.w_qnorm: Optional[torch.Tensor] = None
        self.w_in: Optional[torch.Tensor] = None            # [H (dn + dr) + rank + dr + H dv, hidden]
        self.w_norm: Optional[torch.Tensor] = None
        self.w_uk_t: Optional[torch.Tensor] = None          # [H, rank, dn]
        self.w_uv: Optional[torch.Tensor] = None            # [H, dv, rank]

    # ---- what it needs ---------------------------------------------------
    def weights(self) -> Dict[str, WeightSpec]:
        H, W, dn, dr, dv, rank, nm = self.nh, self.hidden_size, self.dn, self.dr, self.dv, self.rank, self.names
        init = ("normal", self.init_std)
        out = {} if self.q_rank else {nm["q"]: WeightSpec((H * (dn + dr), W), init)}
        out.update({
            nm["dkv"]: WeightSpec((rank + dr, W), init),
            nm["dkv_norm"]: WeightSpec((rank,), ("uniform", 0.5, 1.5), follows_compute_dtype=False),
            nm["uk"]: WeightSpec((H * dn, rank), ("normal", self.init_std * 4)),
            nm["uv"]: WeightSpec((H * dv, rank), ("normal", self.init_std * 4)),
            nm["o"]: WeightSpec((W, H * dv), init),
        })
        if self.q_rank:
            out[nm["dq"]] = WeightSpec((self.q_rank, W), init)
            out[nm["dq_norm"]] = WeightSpec((self.q_rank,), ("uniform", 0.5, 1.5), follows_compute_dtype=False)
            out[nm["uq"]] = WeightSpec((H * (dn + dr), self.q_rank), ("normal", self.init_std * 4))
        if self.gate:
            out[nm["g"]] = WeightSpec((H * dv, W), init)
        if self.sink:
            out[nm["sink"]] = WeightSpec((H,), ("uniform", -1.0, 1.0), follows_compute_dtype=False)
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        H, dn, dr, dv, rank, nm = self.nh, self.dn, self.dr, self.dv, self.rank, self.names
        wq, wdkv = tensors[nm["uq"] if self.q_rank else nm["q"]], tensors[nm["dkv"]]
        perm = self.position.head_permutation()
        if perm is not None:
            # the encoding's own pairs become the kernels' half-split pairs: the rotated rows of every head's query
            # and of the shared key part change places alike, which no score notices
            p = perm[: self.position.rotary_dim].to(wq.device).long()
            if sorted(p.tolist()) != list(range(self.position.rotary_dim)):
                raise ValueError("the position encoding's head_permutation does not keep the rotated values together")
            wq = wq.clone().view(H, dn + dr, -1)
            wq[:, dn: dn + p.numel()] = wq[:, dn + p]
            wq = wq.reshape(H * (dn + dr), -1)
            wdkv = wdkv.clone()
            wdkv[rank: rank + p.numel()] = wdkv[rank + p]
        if self.q_rank:
            # one product for the two latents (and the gate); the queries' own matrix works on the normed latent
            rows = [tensors[nm["dq"]], wdkv] + ([tensors[nm["g"]]] if self.gate else [])
            self.w_uq = wq.contiguous()
            self.w_qnorm = tensors[nm["dq_norm"]].contiguous()
        else:
            rows = [wq, wdkv] + ([tensors[nm["g"]]] if self.gate else [])
        if self.sink:
            self.sinks = tensors[nm["sink"]].to(torch.float32).contiguous()
        self.w_in = torch.cat(rows, dim=0).contiguous()
        self.w_norm = tensors[nm["dkv_norm"]].contiguous()
        self.w_uk_t = tensors[nm["uk"]].view(H, dn, rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[nm["uv"]].view(H, dv, rank).contiguous()
        self.w_o = tensors[nm["o"]].contiguous()
        prepare_weights(self.rt, [(self.w_in, None, False), (self.w_o, None, True)]
                        + ([(self.w_uq, None, False)] if self.q_rank else []))

    # ---- one step --------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: CacheView):
        H, dn, dr, dv, rank, d = self.nh, self.dn, self.dr, self.dv, self.rank, self.d
        if cache.k_pages is None:
            raise K.KernelError("latent attention needs pages of the cache")
        n = x.shape[0]
        proj = first = linear(x, self.w_in, kernels=self.rt.kernels)
        rows = torch.empty((n, (H + 2) * d), dtype=x.dtype, device=x.device)
        if self.q_rank:             # first: [query latent | latent | rotated key part | gate]
            cq = K.rms_rows(first, 0, self.q_rank, self.w_qnorm, self.norm_eps)
            proj = linear(cq, self.w_uq, kernels=self.rt.kernels)
            K.latent_prepare(proj, rows, self.w_norm, self.norm_eps, H, dn, dr, rank, latent=first, latent_col=self.q_rank)
        else:
            K.latent_prepare(proj, rows, self.w_norm, self.norm_eps, H, dn, dr, rank)
        K.gemm_heads(proj, 0, dn + dr, self.w_uk_t, rows, dr, d)               # Uk_h^T q_plain_h beside rope's part
        attended = self.rotate_attend(rows, ctx, cache, transformed=False)      # [n, H d]: (unused | mixed latents)
        mixed = torch.empty((n, H * dv), dtype=x.dtype, device=x.device)
        K.gemm_heads(attended, dr, d, self.w_uv, mixed, 0, dv,
                     gate=first if self.gate else None,
                     gate_offset=(self.q_rank if self.q_rank else H * (dn + dr)) + rank + dr)
        return linear(mixed, self.w_o, keep_split=True, kernels=self.rt.kernels)

    def native(self, program, view: CacheView) -> None:
        if (type(self).forward is not LatentAttention.forward or type(self).attend is not Attention.attend
                or type(self).rotate_attend is not Attention.rotate_attend):
            return super(Attention, self).native(program, view)
        from ..engine.program import ALWAYS, STREAM, Alt, Value
        if view is None or view.k_pages is None or view.v_pages is None:
            raise K.KernelError("latent attention needs pages of the cache")
        H, dn, dr, dv, rank, d, rt = self.nh, self.dn, self.dr, self.dv, self.rank, self.d, self.rt
        T, N, act, esz = program.T, program.N, program.act_code, program.act_bytes
        in_row, row = int(self.w_in.shape[0]), (H + 2) * d
        program.keep(self.w_in, self.w_norm, self.w_uk_t, self.w_uv, self.w_o, self.w_uq, self.w_qnorm)
        proj = first = emit_linear(program, program.x, N, self.w_in, rt.dtype, None, False, "latent.proj", "latent.in").tensor()
        rows = program.buffer("latent.rows", T * row * esz)
        q_row, lat, lat_row = in_row, None, 0
        if self.q_rank:
            cq = program.buffer("latent.cq", T * self.q_rank * esz)
            program.op("core", "ia_rms_rows", [first, in_row, self.w_qnorm, K.DTYPE_CODE[self.w_qnorm.dtype], cq,
                                               self.q_rank, act, N, self.q_rank, float(self.norm_eps), STREAM])
            proj = emit_linear(program, cq, N, self.w_uq, rt.dtype, None, False, "latent.q", "latent.uq").tensor()
            q_row, lat, lat_row = H * (dn + dr), first.at(self.q_rank * esz), in_row
        program.op("core", "ia_latent_prepare", [proj, q_row, lat, lat_row, rows, row, act, self.w_norm,
                                                 K.DTYPE_CODE[self.w_norm.dtype], N, H, dn, dr, rank,
                                                 float(self.norm_eps), STREAM])
        program.op("core", "ia_gemm_heads", [proj, q_row, dn + dr, self.w_uk_t, rows.at(dr * esz), row, d,
                                             None, 0, act, N, H, rank, dn, STREAM])
        attended = self.emit_rotate_attend(program, view, Value(row, [Alt(ALWAYS, rows, 0, rt.dtype)]), row)
        mixed = program.buffer("latent.mixed", T * H * dv * esz)
        gate = first.at(((self.q_rank if self.q_rank else H * (dn + dr)) + rank + dr) * esz) if self.gate else None
        program.op("core", "ia_gemm_heads", [attended.at(dr * esz), H * d, d, self.w_uv, mixed, H * dv, dv,
                                             gate, in_row if self.gate else 0, act, N, H, dv, rank, STREAM])
        program.pending = emit_linear(program, mixed, N, self.w_o, rt.dtype, None, True, "latent.mix", "latent.o")


register_part("mixer", "latent_attention", LatentAttention)
